"""Parity of the HIP path (through the C ABI) with the CPU oracle.

Bars: bit-exact for to_float, the activation quantisers, top-k indices, routing weights and the
per-expert token lists; max-abs error <= 2e-3 * rms(output) for block outputs (f32).
"""
import numpy as np
import pytest

import candle_amd
import pyoracle as O
from helpers import CONFIGS, activations, make_pair, make_weights, rms

pytestmark = pytest.mark.gpu

TOL = 2e-3  # max-abs error relative to rms(output), the bar at the benchmark shapes


def block_tol(dt, F):
    """Max-abs tolerance relative to rms(output) for a block of intermediate width F.

    Q4_0 / Q8_0: the first product is bit-identical to the scalar reference, so the re-quantised
    intermediate is too and only the f32 order of the second product differs -> 2e-3 everywhere.
    Q2K ... Q6K: the reference adds eight interleaved partial sums per super-block, the MFMA path one; the
    two differ in the last ulp, which now and then flips one rounding of the re-quantised
    intermediate.  One flipped quant moves an output by (amax/127)*|w2|, i.e. about
    (5/127)/sqrt(F) of rms(output): 3e-4 at F = 14336 (inside 2e-3) but 1.2e-3 at F = 1024, so
    the bar is widened by sqrt(14336/F) for the reduced shapes used here.
    """
    if dt not in (O.Q2K, O.Q3K, O.Q4K, O.Q5K, O.Q6K):   # every format with Q8K activations shares the mechanism
        return TOL
    return TOL * max(1.0, float(np.sqrt(14336.0 / F)))


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def test_device_is_gfx950():
    assert candle_amd.device_arch().startswith("gfx950")


@pytest.mark.parametrize("dt", [O.Q4_0, O.Q4_1, O.Q5_0, O.Q5_1, O.Q8_0, O.Q2K, O.Q3K, O.Q4K, O.Q5K, O.Q6K, O.Q8K])
def test_to_float_bit_exact(dt):
    n = 256 * 96
    x = O.fill_normal(dt, n, 0.0, 0.02)
    x[:256] = 0.0  # an all-zero block
    x[256:512] *= 1e-3  # tiny values: f16 subnormal scales
    x[512] = 3.0  # outlier
    blocks = O.quantize(dt, x)
    assert np.array_equal(bits(candle_amd.dequantize(dt, blocks, n)), bits(O.dequantize(dt, blocks, n)))
    # arbitrary bit patterns in the quant payload (scale fields kept finite)
    rng = np.random.default_rng(dt)
    raw = blocks.copy().reshape(-1, O.BLOCK_BYTES[dt])
    lo, hi = {O.Q4_0: (2, 18), O.Q4_1: (4, 20), O.Q5_0: (2, 22), O.Q5_1: (4, 24), O.Q8_0: (2, 34), O.Q2K: (0, 80), O.Q3K: (0, 108), O.Q4K: (4, 144), O.Q5K: (4, 176), O.Q6K: (0, 208), O.Q8K: (4, 292)}[dt]
    raw[:, lo:hi] = rng.integers(0, 256, raw[:, lo:hi].shape, dtype=np.uint8)
    raw = raw.reshape(-1)
    assert np.array_equal(bits(candle_amd.dequantize(dt, raw, n)), bits(O.dequantize(dt, raw, n)))
    assert candle_amd.dequantize(dt, raw[:0], 0).size == 0


@pytest.mark.parametrize("dt", [O.Q4_0, O.Q8_0, O.Q2K, O.Q3K, O.Q4K, O.Q5K, O.Q6K])
def test_weight_quantiser_bit_exact(dt, golden):
    n = 256 * 2048
    x = O.fill_normal(40 + dt, n, 0.0, 0.02)
    x[:256] = 0.0                  # all-zero super-block
    x[256:288] = 0.0125            # constant sub-block (max == min)
    x[512:768] = np.abs(x[512:768])  # all positive: min clamps to zero
    x[1024:1280] *= 1e-4           # f16-subnormal scales
    x[2048] = 1.0                  # outlier
    assert np.array_equal(candle_amd.quantize_weights(dt, x), O.quantize(dt, x))
    ramp = np.arange(128, dtype=np.float32)
    if dt == O.Q4_0:  # candle-core/tests/quantized_tests.rs:262-291
        got = candle_amd.dequantize(dt, candle_amd.quantize_weights(dt, ramp), 128)
        assert np.array_equal(bits(got), bits(np.array(golden["q4_0_roundtrip_0_127"]["expected"], dtype=np.float32)))
    import torch
    xd = torch.from_numpy(x).cuda()
    out = candle_amd.quantize_weights(dt, xd)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), O.quantize(dt, x))


@pytest.mark.parametrize("vdt", [O.Q8_0, O.Q8_1, O.Q8K])
def test_activation_quantiser_bit_exact(vdt):
    rows, k = 37, 2048
    x = O.fill_normal(5 + vdt, rows * k).reshape(rows, k)
    x[0] = 0.0                      # all-zero row
    x[1, :256] = 0.0                # zero block inside a row
    x[2, 7] = -9.5                  # negative maximum
    x[3, 300] = 9.5                 # positive maximum (maps to -128)
    x[4, 10] = 4.25; x[4, 20] = -4.25  # equal magnitudes: the first one decides the sign
    x[5] *= 1e-20
    x[6] *= 1e20
    x[7, ::2] = 0.5                 # exact .5 ties after scaling
    x[8, :32] = 3.0                 # block sum 32 * 127 = 4064 is not representable in f16 (Q8_1's s rounds it)
    x[9] *= 1e-7                    # Q8_1: s = f16(sum) * d falls among the f16 subnormals
    # scale 1 (the largest magnitude is 128 for Q8K, 127 for Q8_0 / Q8_1): every product is the value itself; halves
    # and their float neighbours on both sides, positive and negative (round() is half away from zero)
    big = 128.0 if vdt == O.Q8K else 127.0
    halves = (np.arange(k) % 120).astype(np.float32) + 0.5
    for row, vals in ((10, halves), (11, -halves), (12, np.nextafter(halves, np.float32(0))), (13, np.nextafter(halves, np.float32(200))),
                      (14, -np.nextafter(halves, np.float32(0))), (15, -np.nextafter(halves, np.float32(200)))):
        x[row] = vals
        x[row, ::32] = -big         # the first element of every block sets the scale (and, for Q8K, the sign)
    got = candle_amd.quantize_act(vdt, x)
    want = O.quantize(vdt, x)
    assert np.array_equal(got, want)
    assert candle_amd.quantize_act(vdt, x[:0]).size == 0


@pytest.mark.parametrize("T,E,k,norm", [(16, 8, 2, True), (1, 8, 2, True), (333, 60, 4, True), (4096, 8, 2, True),
                                         (65, 64, 6, False), (7, 3, 3, True), (50, 160, 8, True), (9, 1, 1, True),
                                         (33, 256, 16, True), (12, 65, 3, False), (20, 100, 5, True), (40, 224, 1, True),
                                         # more than 16384 assignments: the dispatch pass as two launches of several workgroups
                                         (3000, 128, 8, True), (5000, 60, 6, False), (2100, 256, 16, True), (40000, 8, 2, True)])
def test_route_bit_exact_given_logits(T, E, k, norm):
    logits = O.fill_normal(T * 31 + E, T * E, 0.0, 1.5).reshape(T, E)
    if T > 4:
        logits[1] = 0.25            # all tied: experts 0..k-1 must win
        logits[2, E // 2:] = logits[2, : E - E // 2][::-1]  # pairwise ties
        logits[3] = -80.0 * np.arange(E)  # probabilities underflow to zero past the first few
    gi, gw, goff, gperm, gpw = candle_amd.route(logits, k, norm)
    ri, rw, roff, rperm, rpw = O.route(O.softmax_last_dim(logits), k, norm)
    assert np.array_equal(gi, ri)
    assert np.array_equal(bits(gw), bits(rw))
    assert np.array_equal(goff, roff)
    assert np.array_equal(gperm, rperm)
    assert np.array_equal(bits(gpw), bits(rpw))


def test_route_zipf_bias_lists():
    # prefill-like: 4096 tokens, heavy skew
    T, E, k = 4096, 8, 2
    logits = O.fill_normal(99, T * E, 0.0, 1.0).reshape(T, E) + np.log(1.0 / np.arange(1, E + 1)).astype(np.float32) * 2
    gi, gw, goff, gperm, gpw = candle_amd.route(logits, k)
    ri, rw, roff, rperm, rpw = O.route(O.softmax_last_dim(logits), k)
    assert np.array_equal(gi, ri) and np.array_equal(goff, roff) and np.array_equal(gperm, rperm)
    assert goff[1] - goff[0] > 2 * (goff[-1] - goff[-2])


@pytest.mark.parametrize("dt,n,k,m", [(O.Q4K, 64, 512, 5), (O.Q4K, 4096, 1024, 33), (O.Q8_0, 48, 96, 3),
                                       (O.Q2K, 64, 512, 5), (O.Q2K, 1040, 1024, 33), (O.Q2K, 256, 2304, 150),
                                       (O.Q3K, 64, 512, 5), (O.Q3K, 1040, 1024, 33), (O.Q3K, 256, 2304, 150),
                                       (O.Q5K, 64, 512, 5), (O.Q5K, 1040, 1024, 33), (O.Q5K, 256, 2304, 150),
                                       (O.Q6K, 64, 512, 5), (O.Q6K, 1040, 1024, 33), (O.Q6K, 256, 2304, 150),
                                       (O.Q4K, 4096, 1024, 700), (O.Q5K, 4096, 1024, 700), (O.Q6K, 4096, 1024, 700), (O.Q2K, 4096, 1024, 700), (O.Q3K, 4096, 1024, 700),
                                       (O.Q8_0, 4096, 1024, 1100), (O.Q8_0, 2048, 1408, 1100), (O.Q4_0, 4096, 1024, 600), (O.Q5_0, 2048, 1408, 2100),
                                       (O.Q8_0, 256, 1408, 40), (O.Q4_0, 32, 64, 16), (O.Q4_0, 128, 1024, 70),
                                       (O.Q5_0, 48, 96, 3), (O.Q5_0, 256, 1408, 40), (O.Q5_0, 128, 1024, 70),
                                       (O.Q4_1, 48, 96, 3), (O.Q4_1, 256, 1408, 40), (O.Q4_1, 128, 1024, 70),
                                       (O.Q5_1, 48, 96, 3), (O.Q5_1, 256, 1408, 40), (O.Q5_1, 128, 1024, 70)])
def test_qmatmul_against_oracle(dt, n, k, m):
    w = O.fill_normal_quantized(n + k, dt, n, k, 0.02)
    x = activations(m, k, seed=n)
    got = candle_amd.qmatmul(dt, w, n, k, x)
    want = O.matmul(dt, x, w, n)
    if O.BLOCK_ELEMS[dt] == 32:
        # same per-block values added in the same order as the scalar reference loop
        assert np.array_equal(bits(got), bits(want))
    else:
        assert np.abs(got - want).max() <= 1e-5 * rms(want) * 10


def test_q4_0_matmul_known_answers(golden):
    # candle-core/tests/quantized_tests.rs:89-104; four weight rows padded to a 16-row tile
    m, k, n = 3, 64, 4
    lhs = np.arange(m * k, dtype=np.float32).reshape(m, k)
    rhs = np.zeros((16, k), dtype=np.float32)
    rhs[:n] = np.arange(k * n, dtype=np.float32).reshape(n, k)
    got = candle_amd.qmatmul(O.Q4_0, O.quantize(O.Q4_0, rhs), 16, k, lhs)[:, :n]
    assert np.round(got).reshape(-1).tolist() == golden["q4_0_matmul_3_64_4"]["expected_rounded"]


@pytest.mark.parametrize("dt", [O.Q2K, O.Q3K, O.Q4K, O.Q5K, O.Q6K])
def test_few_rows_quantised_inside_the_kernel_equal_the_two_pass_path(dt):
    # up to four rows of a K-quant matrix can take one launch that quantises the rows itself (one or two do by default): same blocks, same products, same
    # order of the partial sums as the row quantiser followed by the streaming kernel -- the same bits -- and the oracle's
    # values.  Shapes: K of 1, 5 and 16 super-blocks (waves with no, one and several blocks), row counts that are not
    # multiples of the workgroups' 32 and 64 rows; rows with an all-zero block and with ties for the largest magnitude.
    for n, k in ((48, 256), (1040, 1280), (16416, 512), (32784, 256), (4096, 4096)):
        w = O.fill_normal_quantized(n + k + dt, dt, n, k, 0.02)
        q = candle_amd.QMatMul(dt, w, n, k)
        try:
            for m in (1, 2, 3, 4):
                x = activations(m, k, seed=100 + m)
                x[0, :256] = 0.0
                if k > 256:
                    x[m - 1, 256:512] = np.where(np.arange(256) % 2 == 0, 1.5, -1.5)   # +-max: the first one sets the sign
                try:
                    candle_amd.set_switch("fused_rows", 2)   # whenever the kernel can: by default three rows take two passes
                    fused = q.forward(x)
                    candle_amd.set_switch("fused_rows", 1)   # never
                    two_pass = q.forward(x)
                finally:
                    candle_amd.set_switch("fused_rows", 0)
                assert np.array_equal(bits(fused), bits(two_pass)), (dt, n, k, m)
                if n * k <= 1040 * 1280:
                    want = O.matmul(dt, x, w, n)
                    assert np.abs(fused - want).max() <= 1e-5 * rms(want) * 10, (dt, n, k, m)
        finally:
            q.close()


@pytest.mark.parametrize("dt", [O.Q8_0, O.Q4_0, O.Q5_0, O.Q4_1, O.Q5_1])
def test_few_rows_of_the_32_element_formats_in_one_launch(dt):
    # the four waves of a workgroup share a row tile's K and one of them adds the block values in ascending block order:
    # the bits of the streaming kernel (one wave per row tile) and of the scalar reference loop.  K of 1, 10, 18 and 32
    # steps of 128 (a wave without blocks, a partial second chunk); a row with an all-zero block.
    for n, k in ((48, 128), (1040, 1280), (256, 2304), (4096, 4096)):
        w = O.fill_normal_quantized(n + k + dt, dt, n, k, 0.02)
        q = candle_amd.QMatMul(dt, w, n, k)
        try:
            for m in (1, 2, 3, 4):
                x = activations(m, k, seed=200 + m)
                x[0, :32] = 0.0
                try:
                    candle_amd.set_switch("fused_rows", 2)
                    fused = q.forward(x)
                    candle_amd.set_switch("fused_rows", 1)
                    two_pass = q.forward(x)
                finally:
                    candle_amd.set_switch("fused_rows", 0)
                assert np.array_equal(bits(fused), bits(two_pass)), (dt, n, k, m)
                if n * k <= 1040 * 1280:
                    assert np.array_equal(bits(fused), bits(O.matmul(dt, x, w, n))), (dt, n, k, m)
        finally:
            q.close()


def test_batch_invariance():
    # qmm_batch, candle-core/tests/quantized_tests.rs:221-256
    n, k = 256, 512
    w = O.fill_normal_quantized(4, O.Q4K, n, k, 0.02)
    x = activations(2, k, seed=8)
    base = candle_amd.qmatmul(O.Q4K, w, n, k, x)
    for reps in (2, 3, 6, 20):
        big = candle_amd.qmatmul(O.Q4K, w, n, k, np.concatenate([x] * reps))
        for r in range(reps):
            assert np.array_equal(bits(big[2 * r: 2 * r + 2]), bits(base))
    # large batches take another kernel (as the reference's CUDA backend does from 9 rows on, where
    # its test allows a summed difference below 1e-4): rows equal each other, and base closely
    n = 4096
    w = O.fill_normal_quantized(5, O.Q4K, n, k, 0.02)
    base = candle_amd.qmatmul(O.Q4K, w, n, k, x)
    big = candle_amd.qmatmul(O.Q4K, w, n, k, np.concatenate([x] * 100))
    for r in range(1, 100):
        assert np.array_equal(bits(big[2 * r: 2 * r + 2]), bits(big[:2]))
    assert np.abs(big[:2] - base).max() <= 1e-4 * rms(base)


def check_block(ref, gpu, T, seed=2, tol=None):
    tol = block_tol(ref.dtype, ref.F) if tol is None else tol
    xs = activations(T, ref.H, seed)
    ys = gpu.forward(xs)
    logits = gpu.last_logits(T)
    # the gate product itself: f32 accumulation order is implementation-defined, values must agree
    _, ref_logits = ref.forward(xs[: min(T, 4)], return_logits=True)
    assert np.abs(logits[: min(T, 4)] - ref_logits).max() < 1e-4
    # routing is bit-exact given the same logits
    gi, gw, goff, gperm, gpw = gpu.last_routing(T)
    ri, rw, roff, rperm, rpw = O.route(O.softmax_last_dim(logits), ref.k, bool(ref.c.norm_topk))
    assert np.array_equal(gi, ri) and np.array_equal(bits(gw), bits(rw))
    assert np.array_equal(goff, roff) and np.array_equal(gperm, rperm) and np.array_equal(bits(gpw), bits(rpw))
    want = ref.forward(xs, logits=logits)
    moe = want - xs if ref.rms_alpha is not None else want
    err = np.abs(ys - want).max()
    assert err <= tol * rms(moe), (err, rms(moe))
    # a wrong term or index moves the whole result, not one element; the flipped quants of a narrow intermediate
    # weigh more (the same sqrt(14336 / F) by which block_tol widens the max-abs bar)
    assert rms(ys - want) <= 2e-4 * (tol / TOL) * rms(moe)
    return ys, want


def test_weight_layout_roundtrip():
    for dt, H, F in ((O.Q4K, 512, 768), (O.Q8_0, 256, 96), (O.Q4_0, 128, 160)):
        ref, gpu = make_pair(H, F, 3, 2, dt, seed=dt, Fs=(64 if dt != O.Q4K else 256))
        for e in range(3):
            for which, src, shape in ((1, ref.w1[e], (F, H)), (3, ref.w3[e], (F, H)), (2, ref.w2[e], (H, F))):
                got = gpu.dequantize_weight(e, which)
                assert np.array_equal(bits(got).reshape(-1), bits(O.dequantize(dt, src, H * F)))
        got = gpu.dequantize_weight(3, 2)
        assert np.array_equal(bits(got).reshape(-1), bits(O.dequantize(dt, ref.sw[2], got.size)))
        gpu.close()


@pytest.mark.parametrize("T", [16, 1, 5])
def test_block_cfg1_q4_0(T):
    c = CONFIGS["cfg1"]
    ref, gpu = make_pair(c["H"], c["F"], c["E"], c["k"], c["dt"], seed=0)
    check_block(ref, gpu, T)
    gpu.close()


@pytest.mark.parametrize("T", [1, 8, 33, 200])
def test_block_q4k_small(T):
    ref, gpu = make_pair(512, 1024, 8, 2, O.Q4K, seed=1)
    check_block(ref, gpu, T)
    gpu.close()


@pytest.mark.parametrize("H", [768, 3072, 5120, 6144, 7168])
def test_block_other_hidden_sizes(H):
    # hidden sizes with their own instantiation of the low-latency front kernel (3072 .. 7168) and one
    # that takes the generic front kernel (768)
    ref, gpu = make_pair(H, 1024, 4, 2, O.Q4K, seed=H)
    for T in (3, 40):
        check_block(ref, gpu, T, tol=block_tol(O.Q4K, 1024))
    gpu.close()


def test_block_q8_0_shared_expert_top4():
    ref, gpu = make_pair(256, 352, 12, 4, O.Q8_0, seed=3, Fs=704)
    check_block(ref, gpu, 40)
    gpu.close()


@pytest.mark.parametrize("T", [20, 40, 70])
def test_block_q4k_shared_expert_slot_tiles(T):
    # the always-on expert sees every token: its streaming kernels carry 2 (T = 20) or 4 (T = 40) 16-slot
    # tiles per pass over the weights, and need a second pass at T = 70
    ref, gpu = make_pair(512, 512, 8, 2, O.Q4K, seed=6, Fs=1024)
    check_block(ref, gpu, T)
    gpu.close()


def test_block_q4k_tile_sizes_and_paths():
    # two slot tiles per streamed pass with a second pass for lists beyond 32 rows (T = 104, 130); from 35 rows per
    # expert the tiled kernel for the up projection with the down projection still streamed, four slot tiles per pass
    # (T = 140, 150, 160, 200, 250), from 65 rows for both: 64-slot tiles (T = 270) up to ~72 rows per expert,
    # 128 beyond (T = 300, 400, 600)
    ref, gpu = make_pair(512, 1024, 8, 2, O.Q4K, seed=1)
    for T in (104, 130, 140, 150, 160, 200, 250, 270, 300, 400, 600):
        check_block(ref, gpu, T)
    gpu.close()


@pytest.mark.parametrize("dt,dt_down", [(O.Q6K, None), (O.Q4K, O.Q6K), (O.Q6K, O.Q4K), (O.Q5K, None), (O.Q5K, O.Q6K),
                                        (O.Q2K, None), (O.Q2K, O.Q4K), (O.Q3K, None), (O.Q3K, O.Q5K)])
def test_block_q6k_and_mixed_down_dtype(dt, dt_down):
    # all-Q6K and all-Q5K experts, the Q4_K_M arrangement (Q4K gate / up with Q6K down), its reverse, and
    # the Q5_K_M arrangement (Q5K with Q6K down).
    # T = 1, 3: narrow workgroups; 8, 33: one and two slot tiles per pass; 70: dispatched lists;
    # 200: a K-quant up projection switches to the tiled kernel; 300, 500: so does such a down projection
    # behind it (64-slot and 128-slot tiles)
    ref, gpu = make_pair(512, 1024, 8, 2, dt, seed=12, dt_down=dt_down)
    for T in (1, 3, 8, 33, 70, 200, 300, 500):
        check_block(ref, gpu, T, tol=block_tol(O.Q4K, 1024))
    for e, which, wdt in ((0, 1, dt), (7, 3, dt), (5, 2, dt_down or dt)):
        want = O.dequantize(wdt, getattr(ref, "w%d" % which)[e], 512 * 1024)
        assert np.array_equal(bits(gpu.dequantize_weight(e, which)).reshape(-1), bits(want))
    gpu.close()


@pytest.mark.parametrize("dt", [O.Q4K, O.Q6K, O.Q2K])
def test_block_kquant_shared_expert_tiny_batches(dt):
    # at most E assignments: the routed experts take the narrow kernels (f32 intermediate, separate quantisation pass),
    # the always-on expert the regular ones
    ref, gpu = make_pair(512, 512, 8, 2, dt, seed=14, Fs=1024)
    for T in (1, 2, 4):
        check_block(ref, gpu, T, tol=block_tol(O.Q4K, 512))
    gpu.close()
    ref, gpu = make_pair(768, 768, 8, 1, dt, seed=15, Fs=1536)
    for T in (1, 8):
        check_block(ref, gpu, T, tol=block_tol(O.Q4K, 768))
    gpu.close()


@pytest.mark.parametrize("dt,dt_down,rms_norm", [(O.Q8_0, None, False), (O.Q4_0, O.Q5_0, True), (O.Q5_1, O.Q4_1, False),
                                                 (O.Q4K, O.Q6K, True), (O.Q5K, None, False), (O.Q3K, O.Q2K, False)])
def test_block_shared_expert_of_a_few_tokens_as_dense_rows(dt, dt_down, rms_norm):
    # one to four tokens: the always-on expert runs as two dense few-row launches (w1 and w3 side by side from the quantised
    # rows, then w2 from silu(w1 x) * (w3 x) quantised in the kernel) instead of the grouped kernels.  Against the oracle in
    # both settings; the 32-element formats add block values in the reference's order either way: same bits.
    legacy = dt in (O.Q8_0, O.Q4_0, O.Q5_1)
    H, F, Fs = (256, 128, 640) if legacy else (512, 256, 1280)
    ref, gpu = make_pair(H, F, 8, 2, dt, seed=70 + dt, Fs=Fs, dt_down=dt_down, rms=rms_norm)
    try:
        for T in (1, 2, 3, 4):
            out = []
            for sw in (2, 1):   # whenever the kernels can / never
                candle_amd.set_switch("fused_rows", sw)
                ys, _ = check_block(ref, gpu, T, seed=T, tol=None if legacy else block_tol(O.Q4K, F))
                out.append(ys)
            if legacy:
                assert np.array_equal(bits(out[0]), bits(out[1]))
    finally:
        candle_amd.set_switch("fused_rows", 0)
    gpu.close()


def test_block_q6k_shared_expert():
    ref, gpu = make_pair(512, 512, 8, 2, O.Q4K, seed=13, Fs=1024, dt_down=O.Q6K)
    for T in (5, 40, 70):
        check_block(ref, gpu, T, tol=block_tol(O.Q4K, 512))
    gpu.close()


@pytest.mark.parametrize("dt,dt_down", [(O.Q5_0, None), (O.Q4_1, None), (O.Q5_1, None), (O.Q4_0, O.Q5_0), (O.Q5_0, O.Q8_0),
                                        (O.Q5_1, O.Q4_1)])
def test_block_legacy_five_bit_and_min_formats(dt, dt_down):
    # Q5_0 (Q8_0 activations, code - 16), Q4_1 and Q5_1 (Q8_1 activations, block minimum times the activation
    # block's s), alone and mixed with another format of the same activation type; with the always-on expert.
    # T = 1, 8: one slot tile; 33: two; 70: a second pass; 300: dispatched lists
    ref, gpu = make_pair(256, 512, 8, 2, dt, seed=31, Fs=256, dt_down=dt_down)
    for T in (1, 8, 33, 70, 300):
        check_block(ref, gpu, T, tol=TOL)
    for e, which, wdt in ((0, 1, dt), (7, 3, dt), (5, 2, dt_down or dt)):
        want = O.dequantize(wdt, getattr(ref, "w%d" % which)[e], 256 * 512)
        assert np.array_equal(bits(gpu.dequantize_weight(e, which)).reshape(-1), bits(want))
    gpu.close()
    # an odd number of 32-element blocks per row and a row count that is not a multiple of 64: the plain kernels
    ref, gpu = make_pair(96, 160, 3, 2, dt, seed=32, dt_down=dt_down)
    for T in (2, 40):
        check_block(ref, gpu, T, tol=TOL)
    gpu.close()


@pytest.mark.parametrize("dt", [O.Q4_0, O.Q4_1, O.Q5_0, O.Q5_1, O.Q8_0])
def test_block_32_element_formats_ragged_row_tiles(dt):
    # The super-tile kernels (K % 128 == 0) run four waves per workgroup behind common barriers; these shapes leave
    # waves without rows: 3 and 5 pairs of row tiles in the up projection (F = 96, 160), 6 row tiles in the down
    # projection (H = 96), and mix super-tile matrices with one-block ones (the other projection's K is not a
    # multiple of 128).
    for H, F in ((128, 96), (128, 160), (96, 256), (384, 640)):
        ref, gpu = make_pair(H, F, 3, 2, dt, seed=40 + H + F, Fs=F)
        for T in (1, 20, 45):
            check_block(ref, gpu, T, tol=TOL)
        gpu.close()
    # dense products with 3 and 5 row tiles, one and three K steps
    for n, k, m in ((48, 128, 3), (80, 384, 40)):
        w = O.fill_normal_quantized(n + k, dt, n, k, 0.02)
        x = activations(m, k, seed=n)
        assert np.array_equal(bits(candle_amd.qmatmul(dt, w, n, k, x)), bits(O.matmul(dt, x, w, n)))


@pytest.mark.parametrize("dt,dt_down", [(O.Q4_0, None), (O.Q5_0, None), (O.Q8_0, None), (O.Q4_0, O.Q8_0), (O.Q5_0, O.Q4_0),
                                        (O.Q4_1, None), (O.Q5_1, None), (O.Q5_1, O.Q4_1)])
def test_block_32_element_formats_tiled_kernels(dt, dt_down):
    # beyond 1024 assignments the slots are grouped by expert and the 32-element formats take the tiled kernels
    # (64-slot tiles): lists of ~300 and ~650 rows, a last tile of every length, and a shared expert beside them
    ref, gpu = make_pair(256, 384, 4, 2, dt, seed=50, dt_down=dt_down)
    for T in (600, 1301):
        check_block(ref, gpu, T, tol=TOL)
    gpu.close()
    ref, gpu = make_pair(128, 256, 6, 3, dt, seed=51, dt_down=dt_down, Fs=384)
    check_block(ref, gpu, 700, tol=TOL)
    gpu.close()
    # a shared expert wide enough for the tiled kernels itself (its tiles follow from the token count, no list)
    ref, gpu = make_pair(128, 256, 6, 3, dt, seed=52, dt_down=dt_down, Fs=1024)
    check_block(ref, gpu, 2100, tol=TOL)
    gpu.close()


def test_mixed_dtypes_need_one_activation_format():
    ref41, _ = make_pair(256, 256, 4, 2, O.Q4_1, seed=6, want_gpu=False)
    with pytest.raises(candle_amd.MoeError, match="quantise activations differently"):   # Q8_1 against Q8_0
        candle_amd.SparseMoeBlock(256, 256, 4, 2, O.Q4_1, ref41.gate, ref41.w1, ref41.w3,
                                  [O.fill_normal_quantized(i, O.Q4_0, 256, 256, 0.02) for i in range(4)], ggml_dtype_down=O.Q4_0)
    ref, _ = make_pair(256, 256, 4, 2, O.Q4_0, seed=6, want_gpu=False)
    with pytest.raises(candle_amd.MoeError, match="quantise activations differently"):
        candle_amd.SparseMoeBlock(256, 256, 4, 2, O.Q4_0, ref.gate, ref.w1, ref.w3,
                                  [O.fill_normal_quantized(i, O.Q6K, 256, 256, 0.02) for i in range(4)], ggml_dtype_down=O.Q6K)


def test_block_no_renorm_and_bias():
    bias = np.log(1.0 / np.arange(1, 9)).astype(np.float32)
    ref, gpu = make_pair(256, 512, 8, 2, O.Q4K, seed=4, norm_topk=False, gate_bias=bias)
    check_block(ref, gpu, 64)
    gpu.close()


@pytest.mark.parametrize("E,k", [(96, 6), (200, 8)])
def test_block_more_than_64_experts(E, k):
    # the front kernel's routing holds up to four experts per lane
    ref, gpu = make_pair(256, 256, E, k, O.Q4K, seed=30 + E)
    for T in (1, 9, 150):
        check_block(ref, gpu, T, tol=block_tol(O.Q4K, 256))
    gpu.close()


@pytest.mark.parametrize("H,E,k,shared,rms", [(2048, 128, 8, 0, False), (2048, 61, 4, 512, False), (4096, 40, 2, 0, False), (2048, 130, 6, 0, True)])
def test_block_dozens_of_experts_at_small_batches(H, E, k, shared, rms):
    # more than 32 experts and rows of 2048 or 4096: all eight waves of the front kernel take gate products (the quantisation
    # of the row is shared out first); with and without the always-on expert's gate row and the pre-norm; 300 tokens take
    # the large-batch variant of the kernel
    ref, gpu = make_pair(H, 256, E, k, O.Q4K, seed=60 + E, Fs=shared, rms=rms)
    for T in (1, 5, 33, 300):
        check_block(ref, gpu, T, tol=block_tol(O.Q4K, 256))
    gpu.close()


@pytest.mark.parametrize("H,E,k,dt,shared,bias", [(512, 8, 2, O.Q4K, 0, False), (2048, 128, 8, O.Q4K, 256, False), (256, 60, 4, O.Q8_0, 64, True),
                                                  (768, 33, 3, O.Q5_1, 0, True)])
def test_block_gate_product_as_a_launch_of_its_own(H, E, k, dt, shared, bias):
    # the front end in two launches (large batches of layers with dozens of experts take it by default: 400 tokens of the
    # 128-expert case): the gate product on the matrix cores -- logits within 1e-4 of the oracle's and of the one-launch
    # kernel's --, then routing (bit-exact given those logits) and quantisation per token
    F = 256 if dt == O.Q4K else 64
    gb = np.random.default_rng(E).normal(0, 0.3, E).astype(np.float32) if bias else None
    ref, gpu = make_pair(H, F, E, k, dt, seed=90 + E, Fs=shared, gate_bias=gb)
    try:
        for T in (1, 17, 400):
            xs = activations(T, H, 2)
            candle_amd.set_switch("front_split", 0)
            gpu.forward(xs)
            one = gpu.last_logits(T)
            candle_amd.set_switch("front_split", 1)
            check_block(ref, gpu, T, tol=block_tol(dt, F))
            assert np.abs(gpu.last_logits(T) - one).max() < 1e-4
            candle_amd.set_switch("front_split", -1)
            if T == 400:
                check_block(ref, gpu, T, tol=block_tol(dt, F))
    finally:
        candle_amd.set_switch("front_split", -1)
    gpu.close()


@pytest.mark.parametrize("E,k,shared", [(60, 4, 64), (16, 3, 0)])
def test_block_dispatch_pass_of_several_workgroups(E, k, shared):
    # more than 16384 assignments: every workgroup of the dispatch pass places its stretch of the assignments behind the
    # earlier ones' and writes its tokens' slots in the order of the combine pass; same result with one workgroup
    T = 16384 // k + 600
    ref, gpu = make_pair(256, 64, E, k, O.Q8_0, seed=95 + E, Fs=shared)
    try:
        ys, _ = check_block(ref, gpu, T)
        candle_amd.set_switch("dispatch_one", 1)
        assert np.array_equal(bits(gpu.forward(activations(T, 256, 2))), bits(ys))
    finally:
        candle_amd.set_switch("dispatch_one", 0)
    gpu.close()


def test_block_rms_residual_chain():
    ref, gpu = make_pair(512, 512, 4, 2, O.Q4K, seed=5, rms=True)
    xs = activations(6, 512, 9)
    for _ in range(3):
        ys = gpu.forward(xs)
        want = ref.forward(xs, logits=gpu.last_logits(6))
        assert np.abs(ys - want).max() <= block_tol(O.Q4K, 512) * rms(want - xs)
        xs = ys
    gpu.close()


@pytest.mark.parametrize("H", [1024, 3072, 4096])
def test_rms_norm_sum_keeps_the_reference_order(H, monkeypatch):
    """rms_norm folds the squares of a row left to right in f32 (candle-nn/src/ops.rs:504-515).  The fast front kernel
    evaluates that fold in chunks (per-chunk significand increments, exact while the running sum stays in one binade);
    the `rms_serial` switch makes it add term by term instead.  Logits and outputs of the two must agree bit for bit on rows
    chosen to stress the chunked form: many exact rounding ties (few mantissa bits), outliers that jump binades, tiny
    terms under a large sum, an all-zero row, a row that overflows to infinity.  The term-by-term form itself is held
    to the oracle by the tolerance tests of the rms-norm layers."""
    ref, gpu = make_pair(H, 256, 4, 2, O.Q4K, seed=6, rms=True)
    rng = np.random.default_rng(H)
    rows = [rng.standard_normal(H),
            rng.integers(-8, 9, H) / 4.0,
            rng.standard_normal(H) * np.exp(3.0 * rng.standard_normal(H)),
            rng.integers(0, 3, H) * 2.0 ** -10,
            np.round(rng.standard_normal(H) * 16) / 16,
            np.zeros(H),
            rng.standard_normal(H) * 1e-20,
            np.full(H, 0.5),
            rng.integers(1, 4, H) * 2.0 ** 60]
    rows[3][rng.integers(0, H, 3)] = 37.5
    rows[8][H // 2] = 1.5e19   # its square is near the top of the f32 range; the sum ends up infinite
    xs = np.ascontiguousarray(np.stack(rows), dtype=np.float32)
    T = xs.shape[0]
    with np.errstate(all="ignore"):
        fast = gpu.forward(xs)
        fast_logits = gpu.last_logits(T)
        candle_amd.set_switch("rms_serial", 1)
        try:
            serial = gpu.forward(xs)
            serial_logits = gpu.last_logits(T)
        finally:
            candle_amd.set_switch("rms_serial", 0)
    assert np.array_equal(bits(fast_logits), bits(serial_logits))
    assert np.array_equal(bits(fast), bits(serial))
    finite = np.isfinite(serial).all(axis=1)
    assert finite[:5].all()
    want = ref.forward(xs[:5], logits=serial_logits[:5])
    assert np.abs(serial[:5] - want).max() <= block_tol(O.Q4K, 256) * rms(want - xs[:5])
    gpu.close()


@pytest.mark.parametrize("dt,T", [(O.Q4K, 1), (O.Q4K, 7), (O.Q4K, 32), (O.Q4K, 100), (O.Q4_0, 16), (O.Q8_0, 300), (O.Q6K, 40), (O.Q5_1, 9)])
def test_top2_outputs_accumulated_in_place_equal_the_combine_pass(dt, T, monkeypatch):
    """With top-2 routing, no shared expert and no residual, the down kernels add a token's two terms into the zeroed
    output row (either order gives the same float) and the combine pass is skipped; the `combine_pass` switch keeps the pass.
    Both must give the same bits, also when the output buffer held other values before the call."""
    torch = pytest.importorskip("torch")
    ref, gpu = make_pair(512, 1024, 8, 2, dt, seed=3)
    xs = activations(T, 512, 31)
    x = torch.from_numpy(xs).cuda()
    out = torch.full_like(x, 7.0)
    gpu.forward(x, out=out)
    torch.cuda.synchronize()
    acc = out.cpu().numpy()
    candle_amd.set_switch("combine_pass", 1)
    try:
        out2 = torch.full_like(x, -3.0)
        gpu.forward(x, out=out2)
        torch.cuda.synchronize()
    finally:
        candle_amd.set_switch("combine_pass", 0)
    assert np.array_equal(bits(acc), bits(out2.cpu().numpy()))
    want = ref.forward(xs, logits=gpu.last_logits(T))
    kquant = dt in (O.Q2K, O.Q3K, O.Q4K, O.Q5K, O.Q6K)   # Q8K activations: the bar of the Q4K blocks at this width
    assert np.abs(acc - want).max() <= block_tol(O.Q4K if kquant else dt, 1024) * rms(want)
    gpu.close()


def test_top2_accumulation_keeps_denormal_terms(monkeypatch):
    # activations of 1e-18 put most outputs below the smallest normal float: the float atomics must not flush them
    torch = pytest.importorskip("torch")
    _, gpu = make_pair(512, 1024, 8, 2, O.Q4K, seed=3, want_gpu=True)
    x = torch.from_numpy((activations(16, 512, 31) * 1e-18).astype(np.float32)).cuda()
    acc, ref_pass = torch.full_like(x, 7.0), torch.full_like(x, 7.0)
    gpu.forward(x, out=acc)
    candle_amd.set_switch("combine_pass", 1)
    try:
        gpu.forward(x, out=ref_pass)
        torch.cuda.synchronize()
    finally:
        candle_amd.set_switch("combine_pass", 0)
    want = ref_pass.cpu().numpy()
    assert ((np.abs(want) < np.finfo(np.float32).tiny) & (want != 0)).sum() > 100
    assert np.array_equal(bits(acc.cpu().numpy()), bits(want))
    gpu.close()


def test_long_inputs_go_through_in_several_passes(monkeypatch):
    # the kernels address quantised rows with 32-bit offsets, so a call carries a bounded number of tokens
    # and longer inputs are cut into passes; forced here at 48 tokens per pass on a 130-token input
    ref, gpu = make_pair(512, 1024, 8, 2, O.Q4K, seed=1)
    xs = activations(130, 512, 21)
    whole = gpu.forward(xs)
    candle_amd.set_switch("max_tokens_per_pass", 48)
    try:
        pieces = gpu.forward(xs)
        with pytest.raises(candle_amd.MoeError):
            gpu.last_logits(130)          # the hooks describe one pass only
        import torch
        dev = gpu.forward(torch.from_numpy(xs).cuda())
        torch.cuda.synchronize()
    finally:
        candle_amd.set_switch("max_tokens_per_pass", 0)
    assert np.array_equal(bits(pieces), bits(dev.cpu().numpy()))
    # a token's result does not depend on which other tokens share its pass, up to the kernel chosen for the
    # pass size (130 tokens: tiled; 48: streamed), hence the tolerance rather than bit equality
    assert np.abs(pieces - whole).max() <= block_tol(O.Q4K, 1024) * rms(whole)
    gpu.forward(xs[:48])
    want = ref.forward(xs[:48], logits=gpu.last_logits(48))
    assert np.abs(pieces[:48] - want).max() <= block_tol(O.Q4K, 1024) * rms(want)
    gpu.close()


def test_large_batch_front_end_and_dispatch_recorded_into_a_hip_graph():
    # 4200 tokens of a 60-expert top-4 layer with an always-on expert: the gate product as a launch of its own, the dispatch
    # pass as two launches of several workgroups -- kernels only, so a capture holds them; replays equal the eager result
    torch = pytest.importorskip("torch")
    ref, gpu = make_pair(256, 64, 60, 4, O.Q8_0, seed=97, Fs=64)
    T = 4200
    xs = [torch.from_numpy(activations(T, 256, 50 + i)).cuda() for i in range(2)]
    eager = [gpu.forward(x).clone() for x in xs]
    x_in, y_out = xs[0].clone(), torch.empty_like(xs[0])
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        gpu.forward(x_in, out=y_out)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        gpu.forward(x_in, out=y_out)
    for rep in range(2):
        for x, want in zip(xs, eager):
            x_in.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_out, want)
            assert torch.equal(gpu.forward(x), want)
    gpu.close()


@pytest.mark.parametrize("T", [4, 32, 200])
def test_forward_recorded_into_a_hip_graph(T):
    # a decode loop records the layer into a graph and replays it: narrow (4), direct (32) and tiled (200)
    # paths; every replay, with eager work and synchronisations in between, must equal the eager result
    torch = pytest.importorskip("torch")
    ref, gpu = make_pair(512, 1024, 8, 2, O.Q4K, seed=1)
    xs = [torch.from_numpy(activations(T, 512, 30 + i)).cuda() for i in range(3)]
    eager = [gpu.forward(x).clone() for x in xs]
    x_in, y_out = xs[0].clone(), torch.empty_like(xs[0])
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        gpu.forward(x_in, out=y_out)            # workspace reserved before the capture
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        gpu.forward(x_in, out=y_out)
    for rep in range(2):
        for x, want in zip(xs, eager):
            x_in.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_out, want)
            assert torch.equal(gpu.forward(x), want)      # eager calls between replays keep working
    # a capture that would have to allocate is refused with a message, not recorded
    big = torch.from_numpy(activations(T + 300, 512, 5)).cuda()
    out = torch.empty_like(big)
    g2 = torch.cuda.CUDAGraph()
    with pytest.raises(candle_amd.MoeError, match="before capturing"):
        with torch.cuda.graph(g2, stream=side):
            gpu.forward(big, out=out)
    torch.cuda.synchronize()
    assert torch.equal(gpu.forward(xs[0]), eager[0])
    # A larger eager forward grows the workspace.  The graph's nodes hold addresses in the old one, which the layer
    # keeps alive from the first capture on: replays after the growth still equal the eager results.
    want_big = gpu.forward(big).clone()
    for x, want in zip(xs, eager):
        x_in.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_out, want)
        assert torch.equal(gpu.forward(big), want_big)
    gpu.close()


def test_top_k_zero_returns_zeros_as_the_reference_does():
    # llama.expert_used_count absent -> n_expert_used = 0 (quantized_llama.rs:507-512): `take(0)` selects nothing
    # (:167) and the block returns zeros; with the fused pre-norm + residual the layer returns its input
    torch = pytest.importorskip("torch")
    for rms_norm in (False, True):
        ref, gpu = make_pair(256, 512, 4, 0, O.Q4K, seed=2, rms=rms_norm)
        xs = activations(9, 256, 4)
        want = ref.forward(xs)
        assert np.array_equal(bits(want), bits(xs if rms_norm else np.zeros_like(xs)))
        assert np.array_equal(bits(gpu.forward(xs)), bits(want))
        out = torch.full((9, 256), 5.0, device="cuda")
        gpu.forward(torch.from_numpy(xs).cuda(), out=out)
        assert np.array_equal(bits(out.cpu().numpy()), bits(want))
        with pytest.raises(candle_amd.MoeError, match="top_k = 0"):
            gpu.last_logits(9)
        gpu.close()
    idx, w, off, perm, pw = candle_amd.route(activations(5, 8, 1), 0)
    assert idx.shape == (5, 0) and not off.any()


@pytest.mark.parametrize("E,k", [(8, 2), (60, 4), (160, 6), (256, 16), (97, 3)])
def test_nan_probabilities_are_ranked_as_total_cmp_ranks_them(E, k):
    """`sort_by(total_cmp)` (quantized_llama.rs:166) puts a NaN with a clear sign bit above every number and one with
    the sign bit set below.  One NaN logit makes the whole softmax row NaN (the sum is NaN), so every key of the row
    is equal and the stable sort keeps index order: experts 0..k-1, with NaN weights."""
    rng = np.random.default_rng(E)
    logits = rng.standard_normal((6, E)).astype(np.float32)
    logits[1, E // 2] = np.float32(np.nan)
    logits[3, 0] = -np.float32(np.nan)
    logits[4, E - 1] = np.float32(np.inf)     # exp(inf - inf) = NaN at that position, exp(-inf) = 0 elsewhere
    with np.errstate(all="ignore"):
        probs = O.softmax_last_dim(logits)
        ri, rw, roff, rperm, rpw = O.route(probs, k)
    gi, gw, goff, gperm, gpw = candle_amd.route(logits, k)
    assert np.array_equal(gi, ri) and np.array_equal(goff, roff) and np.array_equal(gperm, rperm)
    assert np.array_equal(np.isnan(gw), np.isnan(rw))
    ok = ~np.isnan(rw)
    assert np.array_equal(bits(gw)[ok], bits(rw)[ok])
    assert np.isnan(gw[1]).all() and np.array_equal(gi[1], np.arange(k))


@pytest.mark.parametrize("H", [256, 1024, 4096, 1000, 5120])
def test_rms_norm_as_an_operation_of_its_own(H):
    """RmsNorm::forward (quantized_nn.rs:100-126, candle-nn/src/ops.rs:504-515): bit-exact against the oracle, which adds
    the squares left to right as the reference does; with a residual, the sum x + residual is returned as well."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(H)
    x = (rng.standard_normal((11, H)) * np.exp(rng.standard_normal((11, 1)))).astype(np.float32)
    alpha = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    want = O.rms_norm(x, alpha, 1e-5)
    assert np.array_equal(bits(candle_amd.rms_norm(x, alpha, 1e-5)), bits(want))
    xd, ad = torch.from_numpy(x).cuda(), torch.from_numpy(alpha).cuda()
    assert np.array_equal(bits(candle_amd.rms_norm(xd, ad, 1e-5).cpu().numpy()), bits(want))
    res = (rng.standard_normal((11, H)) * 3).astype(np.float32)
    total, y = candle_amd.rms_norm(xd, ad, 1e-5, residual=torch.from_numpy(res).cuda())
    assert np.array_equal(bits(total.cpu().numpy()), bits(x + res))
    assert np.array_equal(bits(y.cpu().numpy()), bits(O.rms_norm(x + res, alpha, 1e-5)))
    with pytest.raises(candle_amd.MoeError):
        candle_amd.rms_norm(x[:, :H - 1], alpha[:H - 1], 1e-5)


def test_shared_expert_layer_recorded_into_a_hip_graph():
    # The always-on expert's kernels run on a side stream of the layer, forked after the front kernels and joined before
    # the combine pass: under stream capture the fork and the join become edges of the graph.
    torch = pytest.importorskip("torch")
    ref, gpu = make_pair(256, 512, 12, 4, O.Q8_0, seed=36, Fs=1024)
    xs = [torch.from_numpy(activations(40, 256, 80 + i)).cuda() for i in range(3)]
    eager = [gpu.forward(x).clone() for x in xs]
    gpu.forward(xs[0])
    assert np.abs(eager[0].cpu().numpy() - ref.forward(xs[0].cpu().numpy(), logits=gpu.last_logits(40))).max() <= 2e-3 * rms(eager[0].cpu().numpy())
    x_in, y_out = xs[0].clone(), torch.empty_like(xs[0])
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        gpu.forward(x_in, out=y_out)
    for rep in range(3):
        for x, w in zip(xs, eager):
            x_in.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_out, w)
            assert torch.equal(gpu.forward(x), w)
    gpu.close()


def test_empty_and_shape_errors():
    ref, gpu = make_pair(256, 256, 4, 2, O.Q4_0, seed=6)
    assert gpu.forward(np.zeros((0, 256), np.float32)).shape == (0, 256)
    assert gpu.forward(np.zeros((2, 3, 256), np.float32)).shape == (2, 3, 256)
    with pytest.raises(candle_amd.MoeError):
        gpu.forward(np.zeros((2, 255), np.float32))
    with pytest.raises(candle_amd.MoeError):
        gpu.forward(np.zeros((2, 256), np.float64))
    gpu.close()
    with pytest.raises(candle_amd.MoeError):
        candle_amd.SparseMoeBlock(256, 256, 4, 5, O.Q4_0, np.zeros((4, 256), np.float32), ref.w1, ref.w3, ref.w2)
    with pytest.raises(candle_amd.MoeError):
        candle_amd.SparseMoeBlock(256, 256, 4, 2, 14, np.zeros((4, 256), np.float32), ref.w1, ref.w3, ref.w2)


def test_device_entry_point_matches_host_entry_point():
    import torch
    ref, gpu = make_pair(512, 1024, 8, 2, O.Q4K, seed=7)
    xs = activations(24, 512, 3)
    y_host = gpu.forward(xs)
    xd = torch.from_numpy(xs).cuda()
    yd = gpu.forward(xd)
    torch.cuda.synchronize()
    assert np.array_equal(bits(yd.cpu().numpy()), bits(y_host))
    gpu.close()


def test_forward_alternating_between_streams():
    # Calls on one layer share its workspace.  On one stream the stream's order serialises them; a call on another
    # stream has to wait for the previous call's kernels (the library records its ordering event only then).
    import torch
    ref, gpu = make_pair(512, 1024, 8, 2, O.Q4K, seed=17)
    xs = [torch.from_numpy(activations(T, 512, 60 + i)).cuda() for i, T in enumerate((40, 3, 40, 17, 64, 5))]
    want = [gpu.forward(x).cpu().numpy() for x in xs]
    streams = [torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.current_stream()]
    torch.cuda.synchronize()
    for rep in range(3):
        outs = []
        for i, x in enumerate(xs):
            st = streams[(i + rep) % 3]
            st.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(st):
                outs.append((st, gpu.forward(x)))
        for (st, y), w in zip(outs, want):
            st.synchronize()
            assert np.array_equal(bits(y.cpu().numpy()), bits(w))
    # the parity hooks wait for the last call wherever it ran
    with torch.cuda.stream(streams[0]):
        y = gpu.forward(xs[0])
    assert gpu.last_logits(40).shape == (40, 8)
    assert np.array_equal(bits(y.cpu().numpy()), bits(want[0]))
    gpu.close()


def test_concurrent_forward_from_several_threads():
    # QuantizedType is Send + Sync (candle-core/src/quantized/mod.rs:256): candle calls a layer from any thread.
    # Four threads share two layers (calls on one layer are serialised inside the library) and use their own inputs.
    import threading
    ref_a, gpu_a = make_pair(512, 1024, 8, 2, O.Q4K, seed=21)
    ref_b, gpu_b = make_pair(256, 512, 8, 2, O.Q8_0, seed=22)
    jobs = [(gpu_a, activations(7, 512, 50)), (gpu_b, activations(33, 256, 51)), (gpu_a, activations(40, 512, 52)), (gpu_b, activations(3, 256, 53))]
    want = [g.forward(x).copy() for g, x in jobs]
    errors, got = [], [None] * len(jobs)

    def work(i):
        try:
            g, x = jobs[i]
            for _ in range(20):
                y = g.forward(x)
                if not np.array_equal(bits(y), bits(want[i])):
                    errors.append("thread %d: result differs from the single-threaded one" % i)
                    return
            got[i] = y
        except Exception as e:  # noqa: BLE001
            errors.append("thread %d: %r" % (i, e))

    ts = [threading.Thread(target=work, args=(i,)) for i in range(len(jobs))]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not errors, errors
    gpu_a.close(); gpu_b.close()


@pytest.mark.parametrize("gate_dt,rms_norm,bias", [(O.Q8_0, False, False), (O.Q4_0, True, True), (O.Q5_1, False, False),
                                                   (O.Q4K, True, False), (O.Q6K, False, True)])
def test_quantised_router(gate_dt, rms_norm, bias):
    # A router tensor that is not F32 / F16 / BF16 stays quantised in the reference (QMatMul::from_arc,
    # quantized/mod.rs:428-447): the logits are k_quants::matmul of the rows the block sees (quantised to the gate dtype's
    # activation format) against the gate's blocks.  Logits against the oracle's matmul (the 32-element formats add their
    # block values in the reference's order: bit for bit), routing bit-exact given the logits, outputs at the usual bar.
    H, F, E, k = 512, 1024, 8, 2
    w1, w3, w2, _ = make_weights(H, F, E, O.Q4K, 61)
    gate = O.fill_normal(6161, E * H, 0.0, 0.02)
    gq = O.quantize(gate_dt, gate)
    gb = O.fill_normal(6162, E, 0.0, 0.5) if bias else None
    alpha = (1.0 + 0.1 * O.fill_normal(6163, H)).astype(np.float32) if rms_norm else None
    ref = O.Layer(H, F, E, k, O.Q4K, None, w1, w3, w2, gate_bias=gb, rms_alpha=alpha, gate_dtype=gate_dt, gate_blocks=gq)
    gpu = candle_amd.SparseMoeBlock(H, F, E, k, O.Q4K, None, w1, w3, w2, gate_bias=gb, rms_alpha=alpha, gate_dtype=gate_dt, gate_blocks=gq)
    for T in (1, 7, 40, 300):
        xs = activations(T, H, 33 + T)
        ys = gpu.forward(xs)
        logits = gpu.last_logits(T)
        want_logits = ref.router_logits(xs)
        if O.BLOCK_ELEMS[gate_dt] == 32:
            assert np.array_equal(bits(logits), bits(want_logits)), (gate_dt, T)
        else:
            assert np.abs(logits - want_logits).max() <= 1e-4 * rms(want_logits), (gate_dt, T)
        gi, gw, goff, gperm, gpw = gpu.last_routing(T)
        ri, rw, roff, rperm, rpw = O.route(O.softmax_last_dim(logits), k)
        assert np.array_equal(gi, ri) and np.array_equal(bits(gw), bits(rw))
        assert np.array_equal(goff, roff) and np.array_equal(gperm, rperm) and np.array_equal(bits(gpw), bits(rpw))
        want = ref.forward(xs, logits=logits)
        moe = want - xs if rms_norm else want
        assert np.abs(ys - want).max() <= block_tol(O.Q4K, F) * rms(moe), (gate_dt, T)
        # the device entry takes the same path
        import torch
        yd = gpu.forward(torch.from_numpy(xs).cuda()).cpu().numpy()
        assert np.array_equal(bits(yd), bits(ys))
    with pytest.raises(candle_amd.MoeError, match="quantised router"):
        import torch
        gpu.forward(torch.from_numpy(activations(4, H, 1)).cuda(), noalloc=True)
    gpu.close()
    with pytest.raises(candle_amd.MoeError, match="multiple of 256"):
        candle_amd.SparseMoeBlock(128, 256, 4, 2, O.Q8_0, None, [np.zeros(128 * 256 // 32 * 34, np.uint8)] * 4, [np.zeros(128 * 256 // 32 * 34, np.uint8)] * 4,
                                  [np.zeros(128 * 256 // 32 * 34, np.uint8)] * 4, gate_dtype=O.Q8_0, gate_blocks=np.zeros(4 * 128 // 32 * 34, np.uint8))
