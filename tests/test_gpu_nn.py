"""The layer-level callers of the path (python/mlx/nn/layers/quantized.py)."""
import pytest
import torch

import mlx_amd
from mlx_amd import nn as qnn
from util import bits_equal

pytestmark = pytest.mark.gpu


def _model(gpu, bias=True):
    return torch.nn.Sequential(
        torch.nn.Embedding(5, 256), torch.nn.ReLU(), torch.nn.Linear(256, 256, bias=bias)
    ).to(gpu)


def test_quantize_swaps_linear_and_embedding(gpu):
    # python/tests/test_nn.py:229-243
    m = qnn.quantize(_model(gpu))
    assert isinstance(m[0], qnn.QuantizedEmbedding)
    assert isinstance(m[1], torch.nn.ReLU)
    assert isinstance(m[2], qnn.QuantizedLinear)
    m = qnn.quantize(_model(gpu), class_predicate=lambda _, mod: isinstance(mod, torch.nn.Linear))
    assert isinstance(m[0], torch.nn.Embedding)
    assert isinstance(m[2], qnn.QuantizedLinear)
    m = qnn.quantize(_model(gpu), class_predicate=lambda p, mod: {"group_size": 32, "bits": 8}
                     if p == "2" else False)
    assert isinstance(m[0], torch.nn.Embedding)
    assert (m[2].group_size, m[2].bits) == (32, 8)
    with pytest.raises(ValueError):
        qnn.quantize(_model(gpu), group_size=64, mode="mxfp4")
    with pytest.raises(ValueError):
        qnn.quantize(_model(gpu), quantize_input=True)


def test_quantized_model_matches_dequantized_dense_model(gpu):
    torch.manual_seed(0)
    dense = _model(gpu)
    q = qnn.quantize(_model(gpu))
    q[0] = qnn.QuantizedEmbedding.from_embedding(dense[0])
    q[2] = qnn.QuantizedLinear.from_linear(dense[2])
    tokens = torch.tensor([[0, 3, 4], [1, 1, 2]], device=gpu)
    got = q(tokens)
    assert got.shape == (2, 3, 256)
    emb = mlx_amd.dequantize(q[0].weight, q[0].scales, q[0].biases)
    w = mlx_amd.dequantize(q[2].weight, q[2].scales, q[2].biases)
    ref = torch.relu(emb[tokens]).double() @ w.double().T + dense[2].bias.detach().double()
    assert float((got.double() - ref).abs().max()) < 1e-4
    # tied output projection
    h = torch.randn(4, 256, device=gpu)
    logits = q[0].as_linear(h)
    assert logits.shape == (4, 5)
    assert float((logits.double() - h.double() @ emb.double().T).abs().max()) < 1e-4


@pytest.mark.parametrize("bits", (2, 3, 4, 5, 6, 8))
def test_quantized_linear_shapes(gpu, bits):
    # python/tests/test_nn.py:268-281: packed width for every code width
    lin = torch.nn.Linear(1536, 1024).to(gpu)
    ql = qnn.QuantizedLinear.from_linear(lin, bits=bits)
    assert ql.weight.shape == (1024, 1536 * bits // 32)
    assert ql.scales.shape == ql.biases.shape == (1024, 1536 // 64)
    assert ql(torch.randn(3, 1536, device=gpu)).shape == (3, 1024)
    assert "bits=%d" % bits in repr(ql)
    fresh = qnn.QuantizedLinear(512, 64, bias=False, group_size=128, bits=bits, device=gpu,
                                dtype=torch.bfloat16)
    y = fresh(torch.randn(2, 7, 512, device=gpu, dtype=torch.bfloat16))
    assert y.shape == (2, 7, 64) and y.dtype == torch.bfloat16


def test_safetensors_triplet_round_trip(tmp_path):
    # a quantized model is stored as (weight U32, scales, biases [, bias]) per layer
    # and loads back bit for bit; strict loading reports extra / missing / misshapen names
    import json
    import struct

    from mlx_amd import nn as qnn

    torch.manual_seed(0)
    model = torch.nn.Sequential(torch.nn.Linear(128, 64), torch.nn.ReLU(), torch.nn.Linear(64, 32, bias=False))
    model = model.cuda().to(torch.bfloat16)
    qnn.quantize(model, group_size=32, bits=4)
    path = tmp_path / "model.safetensors"
    qnn.save_weights(model, str(path))
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
    assert header["__metadata__"] == {"format": "mlx"}
    assert header["0.weight"]["dtype"] == "U32" and header["0.weight"]["shape"] == [64, 16]
    assert header["0.scales"]["dtype"] == "BF16" and header["0.scales"]["shape"] == [64, 4]
    assert sorted(k for k in header if k != "__metadata__") == [
        "0.bias", "0.biases", "0.scales", "0.weight", "2.biases", "2.scales", "2.weight"]

    fresh = torch.nn.Sequential(torch.nn.Linear(128, 64), torch.nn.ReLU(), torch.nn.Linear(64, 32, bias=False))
    fresh = fresh.cuda().to(torch.bfloat16)
    qnn.quantize(fresh, group_size=32, bits=4)
    qnn.load_weights(fresh, str(path))
    for (k, a), (_, b) in zip(model.state_dict().items(), fresh.state_dict().items()):
        assert bits_equal(a, b), k
    x = torch.randn(3, 128, device="cuda", dtype=torch.bfloat16)
    assert torch.equal(model(x), fresh(x))

    with pytest.raises(ValueError, match="Missing 1 parameters"):
        qnn.load_weights(fresh, [(k, v) for k, v in model.state_dict().items() if k != "2.scales"])
    with pytest.raises(ValueError, match="not in model"):
        qnn.load_weights(fresh, list(model.state_dict().items()) + [("3.weight", torch.zeros(1))])
    with pytest.raises(ValueError, match="Expected shape"):
        qnn.load_weights(fresh, [(k, v[:1] if k == "0.bias" else v) for k, v in model.state_dict().items()])
    qnn.load_weights(fresh, [("0.bias", torch.ones(64, dtype=torch.bfloat16))], strict=False)
    assert torch.equal(fresh[0].bias, torch.ones(64, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError, match="Unsupported file extension"):
        qnn.save_weights(model, str(tmp_path / "model.npz"))


@pytest.mark.parametrize("tokens", (3, 80))
def test_switch_glu_matches_per_expert_dense(tokens):
    # every routed (token, expert) pair equals the dense gated MLP of that expert's
    # dequantized weights; 80 tokens x 2 take the sort-by-expert route, 3 x 2 do not
    torch.manual_seed(tokens)
    D, H, E, k = 128, 256, 4, 2
    dt = torch.bfloat16
    glu = qnn.SwitchGLU(D, H, E, group_size=64, bits=4, dtype=dt)
    x = torch.randn(tokens, D, device="cuda", dtype=dt)
    indices = torch.stack([torch.randperm(E, device="cuda")[:k] for _ in range(tokens)]).to(torch.uint32)
    y = glu(x, indices)
    assert tuple(y.shape) == (tokens, k, D)

    def dense(layer, e):
        return mlx_amd.dequantize(layer.weight[e], layer.scales[e], layer.biases[e],
                                  group_size=64, bits=4).double()

    worst = 0.0
    for t in range(tokens):
        for j in range(k):
            e = int(indices[t, j])
            xt = x[t].double()
            up = (dense(glu.up_proj, e) @ xt).to(dt).double()
            gate = (dense(glu.gate_proj, e) @ xt).to(dt).double()
            h = (torch.nn.functional.silu(gate.to(dt)) * up.to(dt)).double()
            want = dense(glu.down_proj, e) @ h
            worst = max(worst, float((y[t, j].double() - want).abs().max()))
    # three bf16 roundings of intermediate activations of magnitude ~1
    assert worst <= 0.05, worst


def test_switch_linear_bias_and_sorted_flag():
    torch.manual_seed(1)
    layer = qnn.QuantizedSwitchLinear(64, 96, 3, bias=True, group_size=32, bits=8, dtype=torch.float16)
    layer.bias.copy_(torch.randn(3, 96, device="cuda", dtype=torch.float16))
    x = torch.randn(6, 1, 64, device="cuda", dtype=torch.float16)
    idx = torch.tensor([0, 0, 1, 2, 2, 2], device="cuda", dtype=torch.uint32)
    a = layer(x, idx, sorted_indices=True)
    b = layer(x, idx, sorted_indices=False)
    assert torch.equal(a, b) and tuple(a.shape) == (6, 1, 96)
    w1 = mlx_amd.dequantize(layer.weight[1], layer.scales[1], layer.biases[1], group_size=32, bits=8)
    want = x[2, 0].double() @ w1.double().T + layer.bias[1].double()
    assert float((a[2, 0].double() - want).abs().max()) <= 2e-2


@pytest.mark.parametrize("rows", (1, 5, 16))
def test_swiglu_block_matches_dense(rows):
    # the gated MLP of dequantized weights; up to 8 rows take the fused gate/up
    # call, 16 rows the three separate products, and both agree with each other
    torch.manual_seed(rows)
    D, H, dt = 256, 512, torch.bfloat16
    mlp = qnn.SwiGLU(D, H, group_size=64, bits=4, dtype=dt)
    x = torch.randn(rows, D, device="cuda", dtype=dt)
    y = mlp(x)
    assert tuple(y.shape) == (rows, D) and y.dtype == dt

    def dense(layer):
        return mlx_amd.dequantize(layer.weight, layer.scales, layer.biases,
                                  group_size=64, bits=4).double()

    gate = (x.double() @ dense(mlp.gate_proj).T).to(dt)
    up = (x.double() @ dense(mlp.up_proj).T).to(dt)
    h = (torch.nn.functional.silu(gate) * up).double()
    want = h @ dense(mlp.down_proj).T
    assert float((y.double() - want).abs().max()) <= 0.05
    separate = mlp.down_proj(torch.nn.functional.silu(mlp.gate_proj(x)) * mlp.up_proj(x))
    assert float((y.double() - separate.double()).abs().max()) <= 0.02
