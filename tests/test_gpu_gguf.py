"""The GGUF expert loader on the GPU: a layer built from a file must behave exactly like the layer built
from the same bytes through moe_layer_create (names and metadata as quantized_llama.rs:506-512, 553-578)."""
import numpy as np
import pytest

import candle_amd
import gguf_writer as W
import pyoracle as O
from helpers import activations, make_weights

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def build(dt, H=512, F=1024, E=8, seed=11):
    w1, w3, w2, _ = make_weights(H, F, E, dt, seed)
    gate = O.fill_normal(seed * 1000003 + 777, E * H, 0.0, 0.02).reshape(E, H)
    return gate, w1, w3, w2


@pytest.mark.parametrize("dt", [O.Q4K, O.Q8_0, O.Q4_0, O.Q5_0, O.Q5_1])
@pytest.mark.parametrize("version", [2, 3])
def test_layer_from_gguf_equals_layer_from_arrays(tmp_path, dt, version):
    H, F, E, k = 512, 1024, 8, 2
    gate, w1, w3, w2 = build(dt)
    path = tmp_path / "moe.gguf"
    W.moe_layer_file(path, 3, gate, w1, w3, w2, dt, k, version=version)
    direct = candle_amd.SparseMoeBlock(H, F, E, k, dt, gate, w1, w3, w2)
    loaded = candle_amd.SparseMoeBlock.from_gguf(str(path), 3)
    assert (loaded.hidden, loaded.ffn, loaded.n_experts, loaded.top_k, loaded.dtype) == (H, F, E, k, dt)
    for T in (1, 9, 70):
        xs = activations(T, H, 40 + T)
        assert np.array_equal(bits(direct.forward(xs)), bits(loaded.forward(xs)))
    want = O.dequantize(dt, w2[5], H * F)
    assert np.array_equal(bits(loaded.dequantize_weight(5, 2)).reshape(-1), bits(want).reshape(-1))
    direct.close(); loaded.close()


def test_router_stored_as_f16_bf16_or_quantised(tmp_path):
    H, F, E, k = 512, 1024, 8, 2
    gate, w1, w3, w2 = build(O.Q4K)
    xs = activations(12, H, 5)
    # F16 router: candle widens it (QMatMul::from_arc dequantises F32 / F16 / BF16 tensors, quantized/mod.rs:429-436)
    p16 = tmp_path / "f16.gguf"
    W.moe_layer_file(p16, 0, gate, w1, w3, w2, O.Q4K, k, gate_dtype=1)
    a = candle_amd.SparseMoeBlock.from_gguf(str(p16), 0)
    b = candle_amd.SparseMoeBlock(H, F, E, k, O.Q4K, gate.astype(np.float16).astype(np.float32), w1, w3, w2)
    assert np.array_equal(bits(a.forward(xs)), bits(b.forward(xs)))
    a.close(); b.close()
    # BF16 router (GgmlDType 30): the upper half of the f32 bits
    gb = (bits(gate) >> 16).astype(np.uint16)
    pb = tmp_path / "bf16.gguf"
    W.moe_layer_file(pb, 0, gate, w1, w3, w2, O.Q4K, k, gate_dtype=30, gate_blocks=gb)
    a = candle_amd.SparseMoeBlock.from_gguf(str(pb), 0)
    b = candle_amd.SparseMoeBlock(H, F, E, k, O.Q4K, (gb.astype(np.uint32) << 16).view(np.float32).reshape(E, H), w1, w3, w2)
    assert np.array_equal(bits(a.forward(xs)), bits(b.forward(xs)))
    a.close(); b.close()
    # Q8_0 router: the reference runs it as a quantised product over Q8_0-quantised rows (the QMatMul::QTensor arm of
    # QMatMul::from_arc, quantized/mod.rs:428-447), which gives other logits than the dequantised gate would
    gq = O.quantize(O.Q8_0, gate.reshape(-1))
    pq = tmp_path / "q8.gguf"
    W.moe_layer_file(pq, 0, gate, w1, w3, w2, O.Q4K, k, gate_dtype=O.Q8_0, gate_blocks=gq)
    a = candle_amd.SparseMoeBlock.from_gguf(str(pq), 0)
    b = candle_amd.SparseMoeBlock(H, F, E, k, O.Q4K, None, w1, w3, w2, gate_dtype=O.Q8_0, gate_blocks=gq)
    ya = a.forward(xs)
    assert np.array_equal(bits(ya), bits(b.forward(xs)))
    assert np.array_equal(bits(a.last_logits(xs.shape[0])), bits(O.matmul(O.Q8_0, xs, gq, E)))
    a.close(); b.close()
    # a dtype no quantised product exists for (Q8_1 = 9 is an activation format)
    pq1 = tmp_path / "q81.gguf"
    W.moe_layer_file(pq1, 0, gate, w1, w3, w2, O.Q4K, k, gate_dtype=9, gate_blocks=np.zeros(E * H // 32 * 36, np.uint8))
    with pytest.raises(candle_amd.MoeError, match="unsupported gate_dtype 9"):
        candle_amd.SparseMoeBlock.from_gguf(str(pq1), 0)


def test_missing_expert_used_count_gives_the_reference_zeros(tmp_path):
    # `llama.expert_used_count` absent -> n_expert_used = 0 (quantized_llama.rs:507-512): the block selects nothing and
    # returns zeros (:167)
    H, F, E, k = 512, 1024, 8, 2
    gate, w1, w3, w2 = build(O.Q4K)
    p = tmp_path / "no_used.gguf"
    W.moe_layer_file(p, 0, gate, w1, w3, w2, O.Q4K, k, expert_keys=False, extra_metadata=[("llama.expert_count", W.U32, E)])
    layer = candle_amd.SparseMoeBlock.from_gguf(str(p), 0)
    assert layer.top_k == 0
    xs = activations(5, H, 6)
    assert not layer.forward(xs).any()
    layer.close()


def test_expert_used_count_of_another_type_counts_as_zero(tmp_path):
    # a string-typed (or u64) `llama.expert_used_count` is not an error in the reference: `to_u32` fails and
    # `unwrap_or(0)` makes it 0 (quantized_llama.rs:507-512), the same layer as with the key absent
    H, F, E, k = 512, 1024, 8, 2
    gate, w1, w3, w2 = build(O.Q4K)
    for i, (vt, v) in enumerate(((W.STRING, "2"), (W.U64, 2))):
        p = tmp_path / ("typed%d.gguf" % i)
        W.moe_layer_file(p, 0, gate, w1, w3, w2, O.Q4K, k, expert_keys=False,
                         extra_metadata=[("llama.expert_count", W.U32, E), ("llama.expert_used_count", vt, v)])
        layer = candle_amd.SparseMoeBlock.from_gguf(str(p), 0)
        assert layer.top_k == 0 and layer.n_experts == E
        assert not layer.forward(activations(5, H, 6)).any()
        layer.close()
    # the expert count itself as a u64: 0 experts to the reference, i.e. the dense arm
    p = tmp_path / "typed_count.gguf"
    W.moe_layer_file(p, 0, gate, w1, w3, w2, O.Q4K, k, expert_keys=False,
                     extra_metadata=[("llama.expert_count", W.U64, E), ("llama.expert_used_count", W.U32, k)])
    with pytest.raises(candle_amd.MoeError, match="expert_count is 0"):
        candle_amd.SparseMoeBlock.from_gguf(str(p), 0)


def test_loader_errors(tmp_path):
    H, F, E, k = 512, 1024, 8, 2
    gate, w1, w3, w2 = build(O.Q4K)
    p = tmp_path / "ok.gguf"
    W.moe_layer_file(p, 0, gate, w1, w3, w2, O.Q4K, k)
    with pytest.raises(candle_amd.MoeError, match=r"cannot find tensor info for blk\.1\.ffn_gate_inp\.weight"):
        candle_amd.SparseMoeBlock.from_gguf(str(p), 1)
    # no expert keys: the reference defaults both counts to 0 (quantized_llama.rs:507-512) and takes the dense arm
    p0 = tmp_path / "dense.gguf"
    W.moe_layer_file(p0, 0, gate, w1, w3, w2, O.Q4K, k, expert_keys=False)
    with pytest.raises(candle_amd.MoeError, match="expert_count is 0"):
        candle_amd.SparseMoeBlock.from_gguf(str(p0), 0)
    # ffn_down in a dtype with another activation format: refused, not silently converted
    pm = tmp_path / "mixed.gguf"
    w2_q8 = [np.zeros(H * F // 32 * 34, np.uint8) for _ in range(E)]
    W.moe_layer_file(pm, 0, gate, w1, w3, w2_q8, O.Q4K, k, down_dtype=O.Q8_0)
    with pytest.raises(candle_amd.MoeError, match="quantise activations differently"):
        candle_amd.SparseMoeBlock.from_gguf(str(pm), 0)
    # an unsupported dtype among the experts (Q8_1 = 9, an activation format)
    pu = tmp_path / "q8_1.gguf"
    w2_q81 = [np.zeros(H * F // 32 * 36, np.uint8) for _ in range(E)]
    W.moe_layer_file(pu, 0, gate, w1, w3, w2_q81, O.Q4K, k, down_dtype=9)
    with pytest.raises(candle_amd.MoeError, match="unsupported ggml_dtype 9"):
        candle_amd.SparseMoeBlock.from_gguf(str(pu), 0)


def test_q4_k_m_layer_with_q6k_down(tmp_path):
    # what Q4_K_M files hold for part of their layers: Q4K ffn_gate / ffn_up, Q6K ffn_down
    H, F, E, k = 512, 1024, 8, 2
    w1, w3, w2, _ = make_weights(H, F, E, O.Q4K, 21, dt_down=O.Q6K)
    gate = O.fill_normal(4242, E * H, 0.0, 0.02).reshape(E, H)
    path = tmp_path / "q4_k_m.gguf"
    W.moe_layer_file(path, 7, gate, w1, w3, w2, O.Q4K, k, down_dtype=O.Q6K)
    loaded = candle_amd.SparseMoeBlock.from_gguf(str(path), 7)
    assert (loaded.dtype, loaded.dtype_down) == (O.Q4K, O.Q6K)
    direct = candle_amd.SparseMoeBlock(H, F, E, k, O.Q4K, gate, w1, w3, w2, ggml_dtype_down=O.Q6K)
    ref = O.Layer(H, F, E, k, O.Q4K, gate, w1, w3, w2, dtype_down=O.Q6K)
    for T in (2, 40):
        xs = activations(T, H, 50 + T)
        ys = loaded.forward(xs)
        assert np.array_equal(bits(ys), bits(direct.forward(xs)))
        want = ref.forward(xs, logits=loaded.last_logits(T))
        assert np.abs(ys - want).max() <= 2e-3 * np.sqrt(14336.0 / F) * np.sqrt(np.mean(want.astype(np.float64) ** 2))
    loaded.close(); direct.close()
