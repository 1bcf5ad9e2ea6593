"""The entry point that allocates nothing (`moe_layer_forward_device_noalloc`): same kernels as
`moe_layer_forward_device`, workspace in the library's file-scope device array.  Outputs must equal the allocating
entry's bit for bit, on calls in a row that shrink and grow (the array keeps the previous call's contents)."""
import numpy as np
import pytest

import candle_amd
import pyoracle as O
from helpers import activations, make_pair, rms

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("shape", ["q4k_top2", "q8_0_shared_top4", "q4k_rms"])
def test_noalloc_entry_equals_the_allocating_entry(shape):
    torch = pytest.importorskip("torch")
    if shape == "q4k_top2":
        ref, gpu = make_pair(512, 1024, 8, 2, O.Q4K, seed=31)
    elif shape == "q8_0_shared_top4":
        ref, gpu = make_pair(256, 512, 12, 4, O.Q8_0, seed=32, Fs=1024)
    else:
        ref, gpu = make_pair(512, 1024, 8, 2, O.Q4K, seed=33, rms=True)
    H = ref.H
    # two calls in a row, the second smaller; then tiny (narrow kernels), large (tiled kernels, dispatch pass), small again
    for i, T in enumerate((40, 7, 1, 300, 3)):
        xs = activations(T, H, 90 + i)
        x = torch.from_numpy(xs).cuda()
        want = gpu.forward(x).cpu().numpy()
        out = torch.full_like(x, 3.0)
        gpu.forward(x, out=out, noalloc=True)
        torch.cuda.synchronize()
        assert np.array_equal(bits(out.cpu().numpy()), bits(want)), (shape, T)
        # the hooks describe the call that ran last, whichever workspace it used
        logits = gpu.last_logits(T)
        oracle = ref.forward(xs, logits=logits)
        moe = oracle - xs if shape == "q4k_rms" else oracle
        assert np.abs(want - oracle).max() <= 2e-3 * np.sqrt(14336 / ref.F) * rms(moe), (shape, T)
    gpu.close()


def test_noalloc_entry_rejects_what_does_not_fit():
    torch = pytest.importorskip("torch")
    ref, gpu = make_pair(512, 1024, 8, 2, O.Q4K, seed=31)
    cap = candle_amd.static_scratch_bytes()
    assert cap == 8 * 1024 * 1024
    T = 4096   # needs 4096 * 2 * (1024 * 4 + 512 * 4 + ...) bytes: far beyond the array
    x = torch.from_numpy(activations(T, 512, 5)).cuda()
    with pytest.raises(candle_amd.MoeError, match="static scratch array holds %d" % cap):
        gpu.forward(x, noalloc=True)
    want = gpu.forward(x[:16].contiguous()).cpu().numpy()
    got = gpu.forward(x[:16].contiguous(), noalloc=True).cpu().numpy()
    assert np.array_equal(bits(got), bits(want))
    gpu.close()


def test_noalloc_entry_under_stream_capture():
    # what the entry is for: recorded into a graph without a warm-up call, replayed with eager work in between
    torch = pytest.importorskip("torch")
    ref, gpu = make_pair(512, 1024, 8, 2, O.Q4K, seed=34)
    xs = [torch.from_numpy(activations(24, 512, 70 + i)).cuda() for i in range(3)]
    x_in, y_out = xs[0].clone(), torch.empty_like(xs[0])
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        gpu.forward(x_in, out=y_out, noalloc=True)
    eager = [gpu.forward(x).clone() for x in xs]
    for rep in range(2):
        for x, want in zip(xs, eager):
            x_in.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_out, want)
            assert torch.equal(gpu.forward(x), want)
    gpu.close()


def test_noalloc_entry_between_allocating_calls_on_three_streams():
    # allocating call on stream A, the entry that allocates nothing on B, allocating call on C: each has to wait for
    # the one before it (they share the layer's side stream and events, and the two allocating calls its workspace)
    torch = pytest.importorskip("torch")
    ref, gpu = make_pair(256, 512, 12, 4, O.Q8_0, seed=35, Fs=1024)
    xs = [torch.from_numpy(activations(T, 256, 40 + i)).cuda() for i, T in enumerate((48, 20, 33))]
    want = [gpu.forward(x).clone() for x in xs]
    streams = [torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    for rep in range(3):
        outs = []
        for i, (x, st) in enumerate(zip(xs, streams)):
            with torch.cuda.stream(st):
                outs.append(gpu.forward(x, noalloc=(i == 1)))
        torch.cuda.synchronize()
        for y, w in zip(outs, want):
            assert torch.equal(y, w), rep
    gpu.close()
