"""Block-level check of the oracle (no reference test exists for the MoE block): the quantised
block must agree with a float64 model that uses the dequantised weights and the same routing,
to within the 8-bit activation-quantisation noise."""
import numpy as np
import pytest


def make_layer(O, H, F, E, k, dt, seed=0, Fs=0, rms=False, norm_topk=True):
    rng = np.random.default_rng(seed)
    q = lambda r, c: O.quantize(dt, rng.normal(0, 0.02, (r, c)).astype(np.float32))
    w1 = [q(F, H) for _ in range(E)]
    w3 = [q(F, H) for _ in range(E)]
    w2 = [q(H, F) for _ in range(E)]
    gate = rng.normal(0, 0.02, (E, H)).astype(np.float32)
    kw = {}
    if Fs:
        kw.update(Fs=Fs, sw1=q(Fs, H), sw3=q(Fs, H), sw2=q(H, Fs), shared_gate=rng.normal(0, 0.02, H).astype(np.float32))
    if rms:
        kw.update(rms_alpha=(1 + 0.1 * rng.normal(0, 1, H)).astype(np.float32), rms_eps=1e-5)
    return O.Layer(H, F, E, k, dt, gate, w1, w3, w2, norm_topk=norm_topk, **kw)


def float64_block(O, L, xs, logits):
    H, F, E, k, dt = L.H, L.F, L.E, L.k, L.dtype
    x_in = xs.astype(np.float64)
    x = x_in
    if L.rms_alpha is not None:
        x = x / np.sqrt((x * x).mean(1, keepdims=True) + L.c.rms_eps) * L.rms_alpha
    probs = O.softmax_last_dim(logits)
    idx, w, *_ = O.route(probs, k, norm_topk=bool(L.c.norm_topk))
    deq = lambda b, r, c: O.dequantize(dt, b, r * c).reshape(r, c).astype(np.float64)
    ys = np.zeros_like(x)
    silu = lambda v: v / (1 + np.exp(-v))
    for e in range(E):
        rows = np.nonzero((idx == e).any(1))[0]
        if rows.size == 0:
            continue
        W1, W3, W2 = deq(L.w1[e], F, H), deq(L.w3[e], F, H), deq(L.w2[e], H, F)
        h = silu(x[rows] @ W1.T) * (x[rows] @ W3.T)
        we = np.array([w[t][idx[t].tolist().index(e)] for t in rows], dtype=np.float64)
        ys[rows] += (h @ W2.T) * we[:, None]
    if L.c.Fs:
        Fs = L.c.Fs
        W1, W3, W2 = deq(L.sw[0], Fs, H), deq(L.sw[1], Fs, H), deq(L.sw[2], H, Fs)
        g = 1 / (1 + np.exp(-(x @ L.shared_gate.astype(np.float64))))
        ys += ((silu(x @ W1.T) * (x @ W3.T)) @ W2.T) * g[:, None]
    if L.rms_alpha is not None:
        ys += x_in
    return ys


@pytest.mark.parametrize("dt,H,F,E,k,T,Fs,rms", [
    (2, 256, 512, 8, 2, 16, 0, False),
    (12, 512, 768, 8, 2, 9, 0, False),
    (8, 256, 384, 12, 4, 21, 512, False),
    (12, 256, 512, 4, 2, 6, 0, True),
])
def test_block_close_to_float64_model(O, dt, H, F, E, k, T, Fs, rms):
    L = make_layer(O, H, F, E, k, dt, seed=dt + T, Fs=Fs, rms=rms)
    xs = np.random.default_rng(99).normal(0, 1, (T, H)).astype(np.float32)
    ys, logits = L.forward(xs, return_logits=True)
    want = float64_block(O, L, xs, logits)
    moe = want - (xs if rms else 0)
    rms = np.sqrt((moe ** 2).mean())
    # 8-bit activations perturb each product by ~0.5-1% of its rms; a dropped term or a wrong
    # index moves the result by O(rms)
    assert np.sqrt(((ys - want) ** 2).mean()) < 0.02 * rms
    assert np.abs(ys - want).max() < 0.1 * rms
    # AVX2 inner loops and threading must not move the result beyond f32 re-association
    ys2 = L.forward(xs, logits=logits, simd=True, threads=4)
    assert np.abs(ys2 - ys).max() < 2e-3 * np.sqrt((moe ** 2).mean())


def test_block_given_logits_and_empty_experts(O):
    L = make_layer(O, 256, 256, 8, 2, 2, seed=5)
    xs = np.random.default_rng(1).normal(0, 1, (4, 256)).astype(np.float32)
    logits = np.zeros((4, 8), dtype=np.float32)
    logits[:, 6] = 5.0
    logits[:, 3] = 4.0  # every token -> experts 6 and 3; the other six experts stay empty
    ys = L.forward(xs, logits=logits)
    want = float64_block(O, L, xs, logits)
    assert np.sqrt(((ys - want) ** 2).mean()) < 0.02 * np.sqrt((want ** 2).mean())
    assert L.forward(xs[:0], logits=logits[:0]).shape == (0, 256)


def test_fill_normal_is_split_invariant(O):
    a = O.fill_normal(3, 100001, 0.0, 0.02, threads=1)
    b = O.fill_normal(3, 100001, 0.0, 0.02, threads=8)
    assert np.array_equal(a, b)
    assert abs(a.std() - 0.02) < 2e-4 and abs(a.mean()) < 2e-4
    q1 = O.fill_normal_quantized(3, O.Q4K, 8, 512, 0.02, threads=4)
    assert np.array_equal(q1, O.quantize(O.Q4K, O.fill_normal(3, 8 * 512, 0.0, 0.02)))


def test_scalar_and_avx2_paths_of_the_reference_flip_requantised_values(O):
    """Context for the block tolerance.  candle's two x86 code paths (vec_dot_unopt and the AVX2
    vec_dot) add the same exact integer block dots in different f32 orders.  The last-ulp difference
    of the first product now and then flips one value of the re-quantised intermediate, and one
    flipped quant moves an output by about (amax/127)*|w2|.  So two *reference* runs already differ
    by a few 1e-3 of rms(output) at the maximum once enough values are involved; measured at
    H=4096, F=14336, 96 rows of one expert: 16 flips in 1.38 M quants, max-abs 2.5e-3 * rms."""
    if not O.lib().orc_has_avx2():
        import pytest
        pytest.skip("no AVX2")
    H, F, T = 1024, 4096, 128
    w1 = O.fill_normal_quantized(1, O.Q4K, F, H, 0.02)
    w3 = O.fill_normal_quantized(2, O.Q4K, F, H, 0.02)
    w2 = O.fill_normal_quantized(3, O.Q4K, H, F, 0.02)
    x = O.fill_normal(9, T * H).reshape(T, H)
    outs = []
    for simd in (False, True):
        a = O.matmul(O.Q4K, x, w1, F, simd=simd, threads=8)
        b = O.matmul(O.Q4K, x, w3, F, simd=simd, threads=8)
        h = ((a / (1 + np.exp(-a.astype(np.float64)))).astype(np.float32) * b).astype(np.float32)
        outs.append((a, O.quantize(O.Q8K, h), O.matmul(O.Q4K, h, w2, H, simd=simd, threads=8)))
    (a0, q0, y0), (a1, q1, y1) = outs
    r = np.sqrt((y0.astype(np.float64) ** 2).mean())
    assert np.abs(a0 - a1).max() <= 1e-5 * np.sqrt((a0.astype(np.float64) ** 2).mean())  # ulp-level only
    flips = int((q0.reshape(-1, 292)[:, 4:260] != q1.reshape(-1, 292)[:, 4:260]).sum())
    diff = np.abs(y0 - y1).max() / r
    # without a flip the two paths agree to 1e-5; every flip shows up as an O(1e-3) outlier
    assert (flips == 0 and diff < 1e-4) or (flips > 0 and 2e-4 < diff < 2e-2)
    assert np.sqrt(((y0 - y1).astype(np.float64) ** 2).mean()) / r < 5e-4


def test_quantised_router_logits_follow_the_quantised_product(O):
    # QMatMul::from_arc (candle-core/src/quantized/mod.rs:428-447) keeps a router tensor of any dtype but F32 / F16 / BF16
    # as a QTensor: logits = k_quants::matmul on the rows the block sees.  Close to the dequantised gate's logits (the
    # gate and the rows are each quantised once), and what forward() routes by when no logits are handed in.
    H, F, E, k = 256, 512, 8, 2
    rng = np.random.default_rng(5)
    gate = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    xs = rng.standard_normal((6, H)).astype(np.float32)
    w = [O.fill_normal_quantized(70 + e, O.Q8_0, F, H, 0.02) for e in range(E)]
    w2 = [O.fill_normal_quantized(80 + e, O.Q8_0, H, F, 0.02) for e in range(E)]
    alpha = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    for dt in (O.Q8_0, O.Q4K):
        gq = O.quantize(dt, gate.reshape(-1))
        layer = O.Layer(H, F, E, k, O.Q8_0, None, w, w, w2, rms_alpha=alpha, gate_dtype=dt, gate_blocks=gq)
        seen = O.rms_norm(xs, alpha, 1e-5)
        lo = layer.router_logits(xs)
        assert np.array_equal(lo, O.matmul(dt, seen, gq, E))
        dense = seen.astype(np.float64) @ O.dequantize(dt, gq, E * H).reshape(E, H).astype(np.float64).T
        assert np.abs(lo - dense).max() < (0.02 if dt == O.Q8_0 else 0.05) * np.abs(dense).max()
        ys, lo2 = layer.forward(xs, return_logits=True)
        assert np.array_equal(lo2, lo)
        assert np.array_equal(ys, layer.forward(xs, logits=lo))
