"""A stack of MoE layers as one call (`moe_stack_forward_device`): the same bits as the layers' own forwards one after
the other, whichever boundaries fold the first layer's combine pass into the second layer's front kernel."""
import numpy as np
import pytest

import candle_amd
import pyoracle as O
from helpers import activations, make_pair, make_weights, rms

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def one_by_one(layers, x):
    h = x
    for layer in layers:
        h = layer.forward(h)
    return h


def build_stack(kinds, H=512, F=1024):
    """kinds: per layer a dict of make_pair options (E, k, dt, rms, Fs, norm_topk)."""
    refs, gpus = [], []
    for i, kw in enumerate(kinds):
        kw = dict(dict(E=8, k=2, dt=O.Q4K, rms=True, Fs=0), **kw)
        ref, gpu = make_pair(H, F, kw["E"], kw["k"], kw["dt"], seed=70 + i, Fs=kw["Fs"], rms=kw["rms"])
        refs.append(ref)
        gpus.append(gpu)
    return refs, gpus


@pytest.mark.parametrize("name,kinds", [
    ("mixtral-like", [{}] * 5),                                                    # every boundary folds
    ("top4 of 12, Q8_0", [dict(E=12, k=4, dt=O.Q8_0)] * 3),
    ("mixed", [{}, dict(rms=False), {}, dict(Fs=512, dt=O.Q8_0), {}, dict(k=1), dict(E=60, k=4), {}]),   # top-2 without a norm accumulates in place; a shared expert keeps its combine pass
    ("no norm at all", [dict(rms=False, k=4, E=8)] * 3),
])
def test_stack_equals_the_layers_one_by_one(name, kinds):
    import torch
    refs, gpus = build_stack(kinds)
    for T in (1, 5, 32, 64, 200, 700):      # decode batches fold; 700 tokens take the dispatch pass and fold nothing
        x = torch.from_numpy(activations(T, 512, 11 + T)).cuda()
        want = one_by_one(gpus, x).cpu().numpy()
        got = candle_amd.stack_forward(gpus, x)
        torch.cuda.synchronize()
        assert np.array_equal(bits(got.cpu().numpy()), bits(want)), (name, T)
        # the hooks still describe every layer's own routing
        for ref, gpu in zip(refs[-1:], gpus[-1:]):
            logits = gpu.last_logits(T)
            gi, gw, goff, gperm, gpw = gpu.last_routing(T)
            ri, rw, roff, rperm, rpw = O.route(O.softmax_last_dim(logits), ref.k)
            assert np.array_equal(gi, ri) and np.array_equal(goff, roff) and np.array_equal(gperm, rperm)
    for gpu in gpus:
        gpu.close()


def test_stack_against_the_oracle_layer_by_layer():
    import torch
    refs, gpus = build_stack([{}] * 4)
    T = 24
    xs = activations(T, 512, 5)
    got = candle_amd.stack_forward(gpus, torch.from_numpy(xs).cuda()).cpu().numpy()
    h = xs
    for ref, gpu in zip(refs, gpus):
        y = gpu.forward(h)                       # the layer alone on the same input: its logits for the oracle
        want = ref.forward(h, logits=gpu.last_logits(T))
        assert np.abs(y - want).max() <= 2e-3 * np.sqrt(14336 / 1024) * rms(want - h)
        h = y
    assert np.array_equal(bits(got), bits(h))
    for gpu in gpus:
        gpu.close()


def test_stack_with_a_quantised_router_and_a_layer_that_selects_nothing():
    import torch
    H, F, E = 512, 1024, 8
    _, a = make_pair(H, F, E, 2, O.Q4K, seed=81, rms=True)
    w1, w3, w2, _ = make_weights(H, F, E, O.Q4K, 82)
    gq = O.quantize(O.Q8_0, O.fill_normal(8282, E * H, 0.0, 0.02))
    alpha = (1.0 + 0.1 * O.fill_normal(8283, H)).astype(np.float32)
    b = candle_amd.SparseMoeBlock(H, F, E, 2, O.Q4K, None, w1, w3, w2, rms_alpha=alpha, gate_dtype=O.Q8_0, gate_blocks=gq)
    c = candle_amd.SparseMoeBlock(H, F, E, 0, O.Q4K, O.fill_normal(8284, E * H, 0.0, 0.02), w1, w3, w2, rms_alpha=alpha)   # top_k = 0
    _, d = make_pair(H, F, E, 2, O.Q4K, seed=83, rms=True)
    layers = [a, b, c, d]
    for T in (3, 40):
        x = torch.from_numpy(activations(T, H, 90 + T)).cuda()
        want = one_by_one(layers, x).cpu().numpy()
        got = candle_amd.stack_forward(layers, x).cpu().numpy()
        assert np.array_equal(bits(got), bits(want)), T
    for layer in layers:
        layer.close()


def test_stack_recorded_into_a_hip_graph_and_called_from_two_streams():
    import torch
    _, gpus = build_stack([{}] * 6)
    xs = [torch.from_numpy(activations(16, 512, 50 + i)).cuda() for i in range(3)]
    eager = [candle_amd.stack_forward(gpus, x).clone() for x in xs]
    for x, want in zip(xs, eager):
        assert torch.equal(one_by_one(gpus, x), want)
    x_in, y_out = xs[0].clone(), torch.empty_like(xs[0])
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        candle_amd.stack_forward(gpus, x_in, out=y_out)
    for rep in range(2):
        for x, want in zip(xs, eager):
            x_in.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_out, want)
            with torch.cuda.stream(side):                    # eager work on another stream between the replays
                assert torch.equal(candle_amd.stack_forward(gpus, x), want)
            assert torch.equal(gpus[2].forward(x), gpus[2].forward(x))
            torch.cuda.synchronize()
    for gpu in gpus:
        gpu.close()


def test_stack_argument_errors():
    import torch
    _, a = make_pair(512, 1024, 8, 2, O.Q4K, seed=91, rms=True)
    _, b = make_pair(256, 512, 8, 2, O.Q4K, seed=92, rms=True)
    x = torch.from_numpy(activations(4, 512, 1)).cuda()
    with pytest.raises(candle_amd.MoeError, match="differ in hidden size"):
        candle_amd.stack_forward([a, b], x)
    with pytest.raises(candle_amd.MoeError, match="appears twice"):
        candle_amd.stack_forward([a, a], x)
    with pytest.raises(candle_amd.MoeError, match="must not alias"):
        candle_amd.stack_forward([a], x, out=x)
    assert torch.equal(candle_amd.stack_forward([a], x), a.forward(x))
    a.close(); b.close()
