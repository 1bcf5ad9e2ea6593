"""Parity at the BASELINE shapes (full sizes).  Weights are drawn on the GPU and quantised with the
library's QTensor::quantize kernels (checked bit-exact against the oracle elsewhere); the same bytes go
to the CPU oracle.  The oracle runs its AVX2 inner loops on all cores here (its scalar loops agree with
them to 1e-6 relative, candle-core/tests/quantized_tests.rs:869-876) to keep the suite short."""
import os

import numpy as np
import pytest

import candle_amd
import pyoracle as O
from helpers import rms

pytestmark = pytest.mark.gpu
TOL = 2e-3
CORES = max(1, min(16, len(os.sched_getaffinity(0))))


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def gpu_weights(dt, rows, cols, n, seed):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    out = []
    for _ in range(n):
        x = torch.randn((rows, cols), generator=g, device="cuda", dtype=torch.float32) * 0.02
        out.append(candle_amd.quantize_weights(dt, x).cpu().numpy())
    return out


def build(H, F, E, k, dt, seed, Fs=0, bias=None, rms_norm=False, norm_topk=True):
    import torch
    w1 = gpu_weights(dt, F, H, E, seed * 10 + 1)
    w3 = gpu_weights(dt, F, H, E, seed * 10 + 2)
    w2 = gpu_weights(dt, H, F, E, seed * 10 + 3)
    g = torch.Generator(device="cuda")
    g.manual_seed(seed * 10 + 4)
    gate = (torch.randn((E, H), generator=g, device="cuda") * 0.02).cpu().numpy()
    okw, gkw = dict(norm_topk=norm_topk, gate_bias=bias), dict(norm_topk=norm_topk, gate_bias=bias)
    if Fs:
        s1, s3 = gpu_weights(dt, Fs, H, 1, seed * 10 + 5)[0], gpu_weights(dt, Fs, H, 1, seed * 10 + 6)[0]
        s2 = gpu_weights(dt, H, Fs, 1, seed * 10 + 7)[0]
        sg = (torch.randn((H,), generator=g, device="cuda") * 0.02).cpu().numpy()
        okw.update(Fs=Fs, sw1=s1, sw3=s3, sw2=s2, shared_gate=sg)
        gkw.update(shared_ffn=Fs, shared_w1=s1, shared_w3=s3, shared_w2=s2, shared_gate=sg)
    if rms_norm:
        alpha = (1.0 + 0.1 * torch.randn((H,), generator=g, device="cuda")).cpu().numpy()
        okw.update(rms_alpha=alpha, rms_eps=1e-5)
        gkw.update(rms_alpha=alpha, rms_eps=1e-5)
    ref = O.Layer(H, F, E, k, dt, gate, w1, w3, w2, **okw)
    gpu = candle_amd.SparseMoeBlock(H, F, E, k, dt, gate, w1, w3, w2, **gkw)
    return ref, gpu


def acts(T, H, seed):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return torch.randn((T, H), generator=g, device="cuda", dtype=torch.float32).cpu().numpy()


def check(ref, gpu, xs, tol=TOL, flip_allowance=False):
    """flip_allowance: for thousands of rows of Q4K the re-quantised intermediate (1e8 values) picks up
    ~1e-5 flipped quants per value -- as two runs of the reference's own scalar and AVX2 paths do
    (tests/test_oracle_block.py) -- and a few outputs land between 2e-3 and 4e-3 of rms.  Then the
    2e-3 bar is required of all but a 1e-4 fraction of the outputs and 4e-3 of every one."""
    T = xs.shape[0]
    ys = gpu.forward(xs)
    logits = gpu.last_logits(T)
    gi, gw, goff, gperm, gpw = gpu.last_routing(T)
    ri, rw, roff, rperm, rpw = O.route(O.softmax_last_dim(logits), ref.k, bool(ref.c.norm_topk))
    assert np.array_equal(gi, ri) and np.array_equal(bits(gw), bits(rw))
    assert np.array_equal(goff, roff) and np.array_equal(gperm, rperm) and np.array_equal(bits(gpw), bits(rpw))
    # Q4_0 / Q8_0: the HIP path adds the block values in vec_dot_unopt's order, so the scalar oracle is the
    # bit-exact partner of the first product; Q4K has no such partner and uses the faster AVX2 loops
    want = ref.forward(xs, logits=logits, simd=(ref.dtype == O.Q4K), threads=CORES)
    moe = want - xs if ref.rms_alpha is not None else want
    err = float(np.abs(ys - want).max())
    if flip_allowance:
        assert err <= 2 * tol * rms(moe), (err, rms(moe), err / rms(moe))
        assert float((np.abs(ys - want) > tol * rms(moe)).mean()) <= 1e-4
    else:
        assert err <= tol * rms(moe), (err, rms(moe), err / rms(moe))
    assert rms(ys - want) <= 2e-4 * rms(moe)
    return ys, roff


@pytest.fixture(scope="module")
def mixtral_layer():
    ref, gpu = build(4096, 14336, 8, 2, O.Q4K, seed=0)
    yield ref, gpu
    gpu.close()


@pytest.mark.parametrize("T", [1, 8, 32, 64])
def test_cfg2_mixtral_q4k_decode(mixtral_layer, T):
    ref, gpu = mixtral_layer
    check(ref, gpu, acts(T, 4096, 100 + T))


def test_cfg2_weight_layout_roundtrip(mixtral_layer):
    ref, gpu = mixtral_layer
    for e, which, src in ((0, 1, ref.w1[0]), (7, 2, ref.w2[7]), (3, 3, ref.w3[3])):
        got = gpu.dequantize_weight(e, which)
        assert np.array_equal(bits(got).reshape(-1), bits(O.dequantize(O.Q4K, src, got.size)))


def test_cfg2_device_entry_and_repeatability(mixtral_layer):
    import torch
    ref, gpu = mixtral_layer
    xs = acts(32, 4096, 7)
    y0 = gpu.forward(xs)
    xd = torch.from_numpy(xs).cuda()
    y1 = gpu.forward(xd).cpu().numpy()
    y2 = gpu.forward(xd).cpu().numpy()
    assert np.array_equal(bits(y0), bits(y1)) and np.array_equal(bits(y1), bits(y2))


ZIPF_BIAS = np.array([0.0, -1.158, -1.581, -1.845, -2.033, -2.186, -2.299, -2.398], dtype=np.float32)


def test_cfg3_prefill_zipf(mixtral_layer):
    # 4096 tokens; a per-expert bias on the logits makes the top-2 load follow Zipf(s=1): shares 1/i,
    # heaviest expert ~37 %.  The biases were fitted once on N(0, 1.28^2) logits (what an N(0, 0.02) gate
    # gives on N(0, 1) activations of width 4096).
    ref, gpu0 = mixtral_layer
    bias = ZIPF_BIAS
    gate = ref.gate
    gpu = candle_amd.SparseMoeBlock(4096, 14336, 8, 2, O.Q4K, gate, ref.w1, ref.w3, ref.w2, gate_bias=bias)
    ref_b = O.Layer(4096, 14336, 8, 2, O.Q4K, gate, ref.w1, ref.w3, ref.w2, gate_bias=bias)
    xs = acts(4096, 4096, 11)
    _, off = check(ref_b, gpu, xs, flip_allowance=True)
    load = np.diff(off) / off[-1]
    zipf = 1.0 / np.arange(1, 9)
    assert np.abs(load - zipf / zipf.sum()).max() < 0.03, load  # the skew really is Zipf(1)
    gpu.close()


def test_cfg4_fine_grained_q8_0_shared_expert():
    ref, gpu = build(2048, 1408, 60, 4, O.Q8_0, seed=4, Fs=5632)
    check(ref, gpu, acts(512, 2048, 12))
    check(ref, gpu, acts(37, 2048, 13))
    gpu.close()


def test_cfg5_chain_rmsnorm_residual():
    """Three chained layers (the full 32 differ only in count), 32-token decode batch, steps with noise.
    After a few residual adds the hidden state is heavy-tailed, the Q8K steps get coarser and a single
    flipped quant of the re-quantised intermediate is worth up to 2e-3 of rms(output): candle's own
    scalar and AVX2 paths then differ from each other by 1.2e-3 .. 2.2e-3 per layer on these inputs.
    The HIP result has to stay within 2e-3 of the reference, or, where the two reference paths are
    further apart than that, no further from either of them than 1.5x their own distance."""
    layers = [build(4096, 14336, 8, 2, O.Q4K, seed=20 + i, rms_norm=True) for i in range(3)]
    x = acts(32, 4096, 30)
    for step in range(2):
        h = x
        for ref, gpu in layers:
            y = gpu.forward(h)
            logits = gpu.last_logits(32)
            want_a = ref.forward(h, logits=logits, simd=True, threads=CORES)   # same input per layer
            want_s = ref.forward(h, logits=logits, simd=False, threads=CORES)
            r = rms(want_s - h)
            e_a, e_s = np.abs(y - want_a).max() / r, np.abs(y - want_s).max() / r
            spread = np.abs(want_a - want_s).max() / r
            assert max(e_a, e_s) <= max(TOL, 1.5 * spread), (e_a, e_s, spread)
            assert min(e_a, e_s) <= 1.25 * TOL
            assert rms(y - want_s) <= 2e-4 * r
            h = y
        x = (h + 0.1 * acts(32, 4096, 40 + step)).astype(np.float32)
    for _, gpu in layers:
        gpu.close()


def test_cfg1_q4_0_reference_plumbing():
    ref, gpu = build(1024, 3584, 8, 2, O.Q4_0, seed=1)
    check(ref, gpu, acts(16, 1024, 14))
    gpu.close()
