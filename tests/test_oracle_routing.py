"""Pins the oracle's softmax / rms-norm / routing.  The reference has tests for the first two
(candle-nn/tests/ops.rs) and none for top-k routing, which is therefore pinned by invariants,
constructed ties and a brute-force restatement of quantized_llama.rs:162-179 in Python."""
import numpy as np
import pytest


def test_softmax_known_answers(O, golden):
    g = golden["softmax_last_dim"]
    x = np.log(np.array(g["input_before_log"], dtype=np.float32))
    y = O.softmax_last_dim(x.reshape(-1, 3)).reshape(2, 2, 3)
    assert np.round(y.astype(np.float64), 4).tolist() == g["expected_round4"]
    s = golden["softmax_stability"]
    assert O.softmax_last_dim(np.array([s["input"]], dtype=np.float32))[0].tolist() == s["expected"]


@pytest.mark.parametrize("E", [8, 31, 32, 60, 64, 96])
def test_softmax_against_float64(O, E):
    rng = np.random.default_rng(E)
    x = rng.normal(0, 2, (64, E)).astype(np.float32)
    y = O.softmax_last_dim(x)
    xd = x.astype(np.float64)
    want = np.exp(xd - xd.max(1, keepdims=True))
    want /= want.sum(1, keepdims=True)
    assert np.abs(y - want).max() < 3e-7
    # the oracle's summation order for E >= 32 is the 4x8-lane order of the AVX2 build; check it
    # against an independent numpy restatement of that order
    e = np.exp((x - x.max(1, keepdims=True)).astype(np.float32), dtype=np.float64).astype(np.float32)
    import ctypes, math
    libm = ctypes.CDLL("libm.so.6"); libm.expf.restype = ctypes.c_float; libm.expf.argtypes = [ctypes.c_float]
    e = np.array([[libm.expf(float(v)) for v in row] for row in (x - x.max(1, keepdims=True)).astype(np.float32)], dtype=np.float32)
    np_ = E & ~31
    tot = np.zeros(64, dtype=np.float32)
    if np_:
        acc = np.zeros((64, 4, 8), dtype=np.float32)
        for i in range(0, np_, 32):
            acc = acc + e[:, i:i + 32].reshape(64, 4, 8)
        x0 = (acc[:, 0] + acc[:, 1]) + (acc[:, 2] + acc[:, 3])
        t0 = x0[:, :4] + x0[:, 4:]
        tot = (t0[:, 0] + t0[:, 1]) + (t0[:, 2] + t0[:, 3])
    for i in range(np_, E):
        tot = tot + e[:, i]
    assert np.array_equal((e / tot[:, None]).view(np.uint32), y.view(np.uint32))


def test_rms_norm_and_sigmoid(O, golden):
    g = golden["rms_norm"]
    x = np.array(g["input"], dtype=np.float32).reshape(-1, 3)
    y = O.rms_norm(x, g["alpha"], g["eps"]).reshape(2, 2, 3)
    assert np.round(y.astype(np.float64), 4).tolist() == g["expected_round4"]
    for v in (3.0, 1.0, 4.0, 5.0, 9.0, -2.5, 0.0):
        assert abs(O.sigmoid(v) - 1 / (1 + np.exp(-v))) < 1e-7
        assert abs(O.silu(v) - v / (1 + np.exp(-v))) < 1e-6


def brute_route(probs, k):
    """Literal Python restatement of quantized_llama.rs:162-179."""
    T, E = probs.shape
    top_x = [[] for _ in range(E)]
    rws = [[] for _ in range(E)]
    for t in range(T):
        rw = probs[t]
        dst = sorted(range(E), key=lambda i: -float(rw[i]))  # Python's sort is stable, like sort_by
        s = np.float32(0)
        for e in dst[:k]:
            s = np.float32(s + rw[e])
            top_x[e].append(t)
        for e in dst[:k]:
            rws[e].append(np.float32(rw[e] / s))
    return top_x, rws


@pytest.mark.parametrize("T,E,k", [(16, 8, 2), (1, 8, 2), (37, 60, 4), (5, 4, 4), (9, 3, 1), (0, 8, 2)])
def test_route_matches_brute_force(O, T, E, k):
    rng = np.random.default_rng(T * 100 + E)
    probs = O.softmax_last_dim(rng.normal(0, 1, (max(T, 1), E)).astype(np.float32))[:T]
    idx, w, offsets, perm, perm_w = O.route(probs.reshape(T, E), k)
    top_x, rws = brute_route(probs.reshape(T, E), k)
    assert offsets[0] == 0 and offsets[-1] == T * k
    for e in range(E):
        lo, hi = offsets[e], offsets[e + 1]
        assert perm[lo:hi].tolist() == top_x[e]
        assert perm_w[lo:hi].view(np.uint32).tolist() == np.array(rws[e], dtype=np.float32).view(np.uint32).tolist()
        assert sorted(top_x[e]) == top_x[e]  # ascending token index
    if T:
        assert np.allclose(w.sum(1), 1.0, atol=3e-7)
        assert all(len(set(r)) == k for r in idx.tolist())


def test_route_ties_pick_lowest_index(O):
    probs = np.full((3, 8), 0.125, dtype=np.float32)
    idx, w, *_ = O.route(probs, 2)
    assert idx.tolist() == [[0, 1]] * 3 and w.tolist() == [[0.5, 0.5]] * 3
    probs = np.array([[0.1, 0.3, 0.3, 0.1, 0.1, 0.1]], dtype=np.float32)
    assert O.route(probs, 3)[0].tolist() == [[1, 2, 0]]
    # against torch.topk on tie-free rows
    import torch
    rng = np.random.default_rng(1)
    p = O.softmax_last_dim(rng.normal(0, 1, (256, 60)).astype(np.float32))
    idx, *_ = O.route(p, 4)
    assert np.array_equal(idx, torch.topk(torch.from_numpy(p), 4, dim=-1).indices.numpy())


def test_route_without_renorm(O):
    rng = np.random.default_rng(2)
    p = O.softmax_last_dim(rng.normal(0, 1, (10, 6)).astype(np.float32))
    idx, w, *_ = O.route(p, 2, norm_topk=False)
    assert np.array_equal(w, np.take_along_axis(p, idx, 1))
