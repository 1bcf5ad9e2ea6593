"""The resident dense projection (the `QMatMul::QTensor` arm, candle-core/src/quantized/mod.rs:428-447,
533-537) against the oracle's `k_quants::matmul`: bit-exact for Q4_0 / Q8_0 (same per-block values
added in the scalar reference's order), a few ulp of rms(output) for Q4K (the reference adds eight
interleaved partial sums per super-block, the GPU one exact integer sum)."""
import numpy as np
import pytest

import candle_amd
import gguf_writer as W
import pyoracle as O
from helpers import activations, rms

pytestmark = pytest.mark.gpu

Q4K_TOL = 1e-4  # max-abs error relative to rms(output)


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def check(dt, got, want):
    if O.BLOCK_ELEMS[dt] == 32:
        assert np.array_equal(bits(got), bits(want))
    else:
        assert np.abs(got - want).max() <= Q4K_TOL * rms(want)


@pytest.mark.parametrize("dt,n,k", [(O.Q4K, 512, 1024), (O.Q4K, 4096, 512), (O.Q4K, 272, 512), (O.Q6K, 528, 768), (O.Q5K, 528, 768), (O.Q2K, 528, 768), (O.Q3K, 528, 768), (O.Q8_0, 256, 1408), (O.Q4_0, 128, 1024),
                                   (O.Q4_1, 128, 1024), (O.Q5_0, 256, 1408), (O.Q5_1, 128, 1024)])
def test_resident_projection_over_batch_sizes(dt, n, k):
    # one object, many calls: decode rows, mid batches, and (Q4K, n % 128 == 0) the tiled kernel
    # at 64- and 128-row tiles with ragged last tiles; shrinking and growing batches reuse the workspace
    w = O.fill_normal_quantized(n * 3 + k, dt, n, k, 0.02)
    lin = candle_amd.QMatMul(dt, w, n, k)
    assert np.array_equal(bits(lin.dequantize()).reshape(-1), bits(O.dequantize(dt, w, n * k)).reshape(-1))
    # (the tiled kernel takes over once its grid fills the chip: from 321 rows at n = 4096, 3009 at n = 512)
    for m in (1, 7, 16, 24, 25, 33, 64, 70, 97, 130, 300, 5) + {512: (3100,), 4096: (330, 1100)}.get(n, ()):
        x = activations(m, k, seed=m + n)
        check(dt, lin.forward(x), O.matmul(dt, x, w, n))
    assert lin.forward(np.zeros((0, k), dtype=np.float32)).shape == (0, n)
    lin.close()
    with pytest.raises(candle_amd.MoeError):
        lin.forward(activations(1, k, seed=1))


@pytest.mark.parametrize("dt", [O.Q8_0, O.Q4_0, O.Q5_0, O.Q4_1, O.Q5_1])
def test_dense_product_on_the_tiled_kernel_of_the_32_element_formats(dt):
    # 1024 x 256: eight row blocks of 128; from 2048 rows on the grid holds a workgroup per CU and the product takes the
    # tiled kernel (64-row tiles, the last one ragged), bit for bit what the reference's loop adds up
    n, k = 1024, 256
    w = O.fill_normal_quantized(7 + dt, dt, n, k, 0.02)
    lin = candle_amd.QMatMul(dt, w, n, k)
    for m in (2100, 2049, 130):
        x = activations(m, k, seed=m + dt)
        assert np.array_equal(bits(lin.forward(x)), bits(O.matmul(dt, x, w, n))), m
    lin.close()


def test_device_entry_equals_host_entry_and_keeps_leading_dims():
    torch = pytest.importorskip("torch")
    dt, n, k = O.Q4K, 384, 768
    w = O.fill_normal_quantized(5, dt, n, k, 0.02)
    lin = candle_amd.QMatMul.from_qtensor(dt, w, n, k)
    for shape in ((1, 1, k), (2, 9, k), (3, 50, k)):
        x = activations(int(np.prod(shape[:-1])), k, seed=shape[1]).reshape(shape)
        host = lin.forward(x)
        dev = lin.forward(torch.from_numpy(x).cuda())
        torch.cuda.synchronize()
        assert dev.shape == shape[:-1] + (n,) and host.shape == dev.shape
        assert np.array_equal(bits(host), bits(dev.cpu().numpy()))


def test_batch_rows_do_not_depend_on_the_batch():
    # qmm_batch (candle-core/tests/quantized_tests.rs:221-256) across the streamed / tiled switch
    dt, n, k = O.Q4K, 256, 512
    w = O.fill_normal_quantized(4, dt, n, k, 0.02)
    lin = candle_amd.QMatMul(dt, w, n, k)
    x = activations(2, k, seed=8)
    base = lin.forward(x)
    for reps in (2, 6, 11):      # 4, 12, 22 rows: streamed kernels, bit-identical rows
        big = lin.forward(np.concatenate([x] * reps))
        for r in range(reps):
            assert np.array_equal(bits(big[2 * r: 2 * r + 2]), bits(base))
    big = lin.forward(np.concatenate([x] * 3200))   # 6400 rows: tiled kernel, identical among themselves
    for r in range(1, 3200, 7):
        assert np.array_equal(bits(big[2 * r: 2 * r + 2]), bits(big[:2]))
    assert np.abs(big[:2] - base).max() <= Q4K_TOL * rms(base)


def test_argument_checks():
    w = O.fill_normal_quantized(1, O.Q8_0, 32, 64, 0.02)
    with pytest.raises(candle_amd.MoeError, match="n % 16"):
        candle_amd.QMatMul(O.Q8_0, w[: 34 * 48], 24, 64)
    with pytest.raises(candle_amd.MoeError):
        candle_amd.QMatMul(7, w, 32, 64)       # Q5_1
    lin = candle_amd.QMatMul(O.Q8_0, w, 32, 64)
    with pytest.raises(candle_amd.MoeError, match="expected"):
        lin.forward(np.zeros((3, 32), dtype=np.float32))


def test_projection_from_gguf(tmp_path):
    # names of quantized_llama.rs:533-547
    H = 512
    mats = {"blk.0.attn_q.weight": (O.Q4K, H, H), "blk.0.attn_k.weight": (O.Q8_0, 128, H), "blk.0.attn_v.weight": (O.Q6K, 128, H),
            "output.weight": (O.Q4_0, 1024, H)}
    blocks = {name: O.fill_normal_quantized(i + 3, dt, n, k, 0.02) for i, (name, (dt, n, k)) in enumerate(mats.items())}
    norm = O.fill_normal(9, H, 1.0, 0.1)
    ts = [(name, dt, (n, k), blocks[name].tobytes()) for name, (dt, n, k) in mats.items()]
    ts.append(("blk.0.attn_norm.weight", 0, (H,), norm.tobytes()))
    path = tmp_path / "proj.gguf"
    W.write_gguf(path, [("general.architecture", W.STRING, "llama")], ts)
    x = activations(40, H, seed=3)
    with candle_amd.GgufFile(str(path)) as g:
        for name, (dt, n, k) in mats.items():
            lin = candle_amd.QMatMul.from_gguf(g, name)
            assert (lin.n, lin.k, lin.dtype) == (n, k, dt)
            check(dt, lin.forward(x), O.matmul(dt, x, blocks[name], n))
        with pytest.raises(candle_amd.MoeError, match="two dimensions"):
            candle_amd.QMatMul.from_gguf(g, "blk.0.attn_norm.weight")
        with pytest.raises(candle_amd.MoeError):
            candle_amd.QMatMul.from_gguf(g, "blk.0.attn_output.weight")
    lin = candle_amd.QMatMul.from_gguf(str(path), "output.weight")   # by path: the file is closed again
    check(O.Q4_0, lin.forward(x[:3]), O.matmul(O.Q4_0, x[:3], blocks["output.weight"], 1024))


@pytest.mark.parametrize("m", [8, 1])
def test_projection_recorded_into_a_hip_graph(m):
    # m = 8: quantiser, table and product recorded; m = 1: the single launch that quantises the row itself
    torch = pytest.importorskip("torch")
    dt, n, k = O.Q4K, 512, 1024
    w = O.fill_normal_quantized(6, dt, n, k, 0.02)
    lin = candle_amd.QMatMul(dt, w, n, k)
    xs = [torch.from_numpy(activations(m, k, seed=60 + i)).cuda() for i in range(3)]
    eager = [lin.forward(x).clone() for x in xs]
    x_in, y_out = xs[0].clone(), torch.empty(m, n, device="cuda")
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        lin.forward(x_in, out=y_out)
    # Eager calls with another row count between the replays: a replay rewrites the routing table in the workspace the
    # eager calls share, so an eager call after it must write the table again (a stale table of 8 rows would have the
    # product of 3 rows write rows 3..7 past its output: the rows behind the output are a canary).
    x3 = torch.from_numpy(activations(3, k, seed=1)).cuda()
    want3 = lin.forward(x3).clone()
    check(dt, want3.cpu().numpy(), O.matmul(dt, x3.cpu().numpy(), w, n))
    out3 = torch.empty(3 + 8, n, device="cuda")
    for rep in range(2):
        for x, want in zip(xs, eager):
            x_in.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_out, want)
            out3.fill_(-7.0)
            lin.forward(x3, out=out3[:3])
            torch.cuda.synchronize()
            assert torch.equal(out3[:3], want3)
            assert bool((out3[3:] == -7.0).all()), "the eager product wrote past its output"
    # a larger eager call moves the workspace to new memory; the graph's nodes keep using the old, which stays alive
    big = torch.from_numpy(activations(m + 300, k, seed=2)).cuda()
    want_big = O.matmul(dt, big.cpu().numpy(), w, n)
    check(dt, lin.forward(big).cpu().numpy(), want_big)
    for x, want in zip(xs, eager):
        x_in.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_out, want)
        check(dt, lin.forward(big).cpu().numpy(), want_big)
    lin.close()


def test_projection_called_from_alternating_streams():
    # Calls on one object share the quantised rows and the routing table: a call on another stream has to wait for
    # the previous call's kernels, or its quantiser overwrites rows the previous product is still reading.
    torch = pytest.importorskip("torch")
    dt, n, k = O.Q4K, 4096, 4096
    w = O.fill_normal_quantized(9, dt, n, k, 0.02)
    lin = candle_amd.QMatMul(dt, w, n, k)
    xs = [torch.from_numpy(activations(m, k, seed=80 + i)).cuda() for i, m in enumerate((64, 3, 200, 17, 64, 5))]
    want = [lin.forward(x).cpu().numpy() for x in xs]
    streams = [torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.current_stream()]
    torch.cuda.synchronize()
    for rep in range(3):
        outs = []
        for i, x in enumerate(xs):
            st = streams[(i + rep) % 3]
            with torch.cuda.stream(st):
                outs.append((st, lin.forward(x)))
        for (st, y), wnt in zip(outs, want):
            st.synchronize()
            assert np.array_equal(bits(y.cpu().numpy()), bits(wnt))
    # the host entry (the object's own stream) after device calls on another stream
    with torch.cuda.stream(streams[0]):
        y = lin.forward(xs[2])
    host = lin.forward(xs[3].cpu().numpy())
    assert np.array_equal(bits(host), bits(want[3]))
    streams[0].synchronize()
    assert np.array_equal(bits(y.cpu().numpy()), bits(want[2]))
    lin.close()
